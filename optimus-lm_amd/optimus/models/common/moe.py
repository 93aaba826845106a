"""optimus.models.common.moe — the fast MoE block, same interface as the reference
(optimus/models/common/moe.py:43-632), computed by the HIP kernels of liboptimus_mi355x.so.

Pipeline of FastOlmoeParallelSparseMoeBlock.forward (reference moe.py:454-621):
  router (softmax -> top-K -> optional renorm)     one wavefront per token          [route.hip]
  K1+K2+K3 index construction                      stable counting sort on device   [sort.hip]
  K4 gather rows into expert order                                                   [rows.hip]
  K5 merged-MLP grouped SwiGLU GEMMs               bf16 MFMA, variable rows/expert  [ggemm.hip]
  K6 weighted combine back to token order                                            [rows.hip]
and the mirrored backward.  There is one code path: the reference's `use_triton_path_*` and
`use_ref_path_*` switches are accepted where its signatures have them and ignored.
"""
import warnings

import torch
import torch.nn as nn
from torch.utils.checkpoint import checkpoint as torch_activation_checkpoint

import pcl_xpu_customops
from optimus import _native as _n
from optimus.profilers import record_pcl_function


# Two of the blocks' fusions only take some operands (see gate_kernel_fits, routed_mlp_kernel_fits);
# for the others the same block runs its unfused sequence of kernels from this library, whose bf16
# roundings fall in other places.  That switch is announced once per reason (a UserWarning), or
# refused when strict_fused_paths is set.
strict_fused_paths = False
_announced_switches = set()


def note_unfused_path(what, why, instead="running the unfused sequence of kernels (same mathematics, bf16 "
                                            "roundings in other places)"):
    """Called where a block leaves a fused kernel path for the unfused sequence."""
    message = f"{what}: {why}; {instead}"
    if strict_fused_paths:
        raise _n.NativeLibraryError(message + " [strict_fused_paths is set]")
    if (what, why) not in _announced_switches:
        _announced_switches.add((what, why))
        warnings.warn(message, stacklevel=3)


def get_tensor_list(tensor, cum_token_counts):
    """Per-expert row slices (reference moe.py:28-35); host-side helper, needs CPU-readable counts."""
    N = len(cum_token_counts) - 1
    return [tensor[cum_token_counts[n]:cum_token_counts[n + 1]] for n in range(N)]


def _device_counts(cum_token_counts, device):
    """The reference hands MergedMLP a CPU int32 tensor (moe.py:494); the kernels read the counts
    from device memory, so accept either and never read them back."""
    if cum_token_counts.device != device:
        cum_token_counts = cum_token_counts.to(device, non_blocking=True)
    if cum_token_counts.dtype != torch.int32:
        cum_token_counts = cum_token_counts.to(torch.int32)
    return cum_token_counts.contiguous()


_single_segment_cache = {}


def single_segment_counts(rows, device):
    """cum_token_counts of one expert that owns all `rows` rows: the device int32 tensor [0, rows],
    built once per (rows, device) so that a dense MLP run through the grouped kernels copies nothing
    from the host per call.  Read-only by contract."""
    key = (int(rows), str(device))
    cum = _single_segment_cache.get(key)
    if cum is None:
        if len(_single_segment_cache) >= 64:
            _single_segment_cache.clear()
        cum = _single_segment_cache[key] = torch.tensor([0, int(rows)], dtype=torch.int32, device=device)
    return cum


def _expert_stride(weight):
    """Elements between consecutive experts of a [G, out, in] weight whose inner two dims are
    dense; 0 for the packed layout."""
    G, o, i = weight.shape
    if weight.stride(2) != 1 or weight.stride(1) != i:
        raise _n.NativeLibraryError("expert weights must be dense [out, in] matrices")
    s = weight.stride(0) if G > 1 else o * i
    return 0 if s == o * i else s


def _require_bf16(*tensors):
    for t in tensors:
        if t.dtype != torch.bfloat16:
            raise TypeError(f"the fused expert kernels run in bfloat16 (got {t.dtype}); cast the "
                            "module with .to(torch.bfloat16)")


def _gemm_dtype(*tensors):
    """bfloat16 (the tuned kernels) or float32 (the plain fp32 kernels) for all operands."""
    dt = tensors[0].dtype
    if dt not in (torch.bfloat16, torch.float32) or any(t.dtype != dt for t in tensors):
        raise TypeError("the grouped expert GEMMs take operands that are all bfloat16 or all float32 "
                        f"(got {[str(t.dtype) for t in tensors]})")
    return dt


def _grouped_gemm(kind, a, b, out, cum, rows, G, N, K, w_stride, accumulate=False):
    """om_grouped_gemm_{fwd,dgrad,wgrad}[_f32][_accumulate] by the operands' dtype; `accumulate`
    (wgrad only) adds the product to `out` in place."""
    suffix = "_f32" if _gemm_dtype(a, b, out) == torch.float32 else ""
    name = f"om_grouped_gemm_{kind}{suffix}" + ("_accumulate" if accumulate else "")
    _n.check(getattr(_n.lib(), name)(_n.ptr(a), _n.ptr(b), _n.ptr(out), _n.ptr(cum), rows, G, N, K,
                                     w_stride, _n.stream()), name)


# ----------------------------------------------------------------------------------------------
# Router
# ----------------------------------------------------------------------------------------------
def gate_kernel_unfit_reason(x, weight):
    """None when the fused gate + routing kernel (om_router_gate_softmax_topk) takes these operands,
    else why not."""
    if not (x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16):
        return f"operands are not bfloat16 device tensors ({x.dtype}, {weight.dtype})"
    N, H = weight.shape
    if N > 256:
        return f"{N} experts (the kernel takes at most 256)"
    if x.shape[0] == 0:
        return "no tokens"
    need = 512 if N <= 64 else 256 if N <= 128 else 64
    if H % need != 0:
        return f"hidden size {H} is not a multiple of {need} (needed with {N} experts)"
    return None


def gate_kernel_fits(x, weight):
    """Shapes and dtypes the fused gate + routing kernel takes (om_router_gate_softmax_topk)."""
    return gate_kernel_unfit_reason(x, weight) is None


def _require_gate_shape(weight, h_multiple, what):
    N, H = weight.shape
    if N > 256 or H % h_multiple != 0:
        raise _n.NativeLibraryError(
            f"{what}: the gate kernels take at most 256 experts and hidden sizes that are multiples "
            f"of {h_multiple} (got {N} experts, hidden {H}); there is no library fallback")


def _gate_weight_grad(x, weight, dlogits):
    """dweight[n,h] = sum_t dlogits[t,n] x[t,h]: a long contraction with a tiny output, split
    over token ranges on the device (om_router_gate_wgrad) instead of a library GEMM that would
    run on a few CUs."""
    _require_gate_shape(weight, 8, "gate weight gradient")
    T, (N, H) = x.shape[0], weight.shape
    lib = _n.lib()
    ws_bytes = lib.om_router_gate_wgrad_workspace_bytes(T, H, N)
    if ws_bytes < 0:
        _n.check(int(ws_bytes), "om_router_gate_wgrad_workspace_bytes")
    workspace = torch.empty(max(int(ws_bytes), 16), dtype=torch.uint8, device=x.device)
    dw = torch.empty_like(weight)
    dlogits = dlogits.contiguous()
    _n.check(lib.om_router_gate_wgrad(_n.ptr(x), _n.ptr(dlogits), T, H, N, _n.ptr(dw), _n.dtype_code(dw),
                                      _n.ptr(workspace), int(ws_bytes), _n.stream()),
             "om_router_gate_wgrad")
    return dw


def _gate_input_grad(weight, dlogits, other_grad=None):
    """dx = bf16(dlogits) @ weight (om_router_gate_dgrad).  With `other_grad` [T,H] (the gradient
    that reached the same hidden states through the experts) the sum of the two is returned, formed
    inside the kernel with autograd's two roundings, so no separate accumulation pass runs."""
    _require_gate_shape(weight, 8, "gate input gradient")
    T, (N, H) = dlogits.shape[0], weight.shape
    dlogits = dlogits.contiguous()
    if other_grad is not None:
        other_grad = other_grad.contiguous()
        _require_bf16(other_grad)
    dx = torch.empty((T, H), dtype=torch.bfloat16, device=dlogits.device)
    _n.check(_n.lib().om_router_gate_dgrad(_n.ptr(dlogits), _n.ptr(weight), _n.ptr(other_grad), _n.ptr(dx),
                                           T, H, N, _n.stream()), "om_router_gate_dgrad")
    return dx


def _gate_backward(x, weight, dlogits, needs, other_grad=None):
    """(dx, dweight) of logits = x @ weight.T for a bf16 gate from the fp32 gradient of the logits,
    rounded to bf16 as it is loaded (the precision a bf16 router's backward has anyway), both on
    bf16 MFMA with fp32 accumulation: om_router_gate_dgrad and om_router_gate_wgrad.  `other_grad`
    is added to dx inside the kernel (see _gate_input_grad)."""
    _require_bf16(x, weight)
    dlogits = dlogits.to(torch.float32)
    dx = dw = None
    if needs[0]:
        dx = _gate_input_grad(weight, dlogits, other_grad)
    if needs[1]:
        dw = _gate_weight_grad(x, weight, dlogits)
    return dx, dw


class GateLogitsFunction(torch.autograd.Function):
    """fp32 logits of a bf16 gate through om_router_gate_logits (one pass over x).  Returns
    (logits, x): the second output is the input itself; a caller that feeds the rest of the layer
    from it makes that part's input gradient arrive here, where the gate's own input gradient is
    added to it inside om_router_gate_dgrad instead of by a separate accumulation pass."""

    @staticmethod
    def forward(ctx, x, weight):
        T, (N, H) = x.shape[0], weight.shape
        logits = torch.empty((T, N), dtype=torch.float32, device=x.device)
        lib = _n.lib()
        if N > 64 or H % 512 != 0:
            # many experts: the weight no longer fits a block's re-reads; split over H instead
            # (also the form for hidden sizes the one-pass kernel does not take)
            ws_bytes = lib.om_router_gate_logits_split_workspace_bytes(T, H, N)
            if ws_bytes < 0:
                _n.check(int(ws_bytes), "om_router_gate_logits_split_workspace_bytes")
            workspace = torch.empty(max(int(ws_bytes), 16), dtype=torch.uint8, device=x.device)
            _n.check(lib.om_router_gate_logits_split(_n.ptr(x), _n.ptr(weight), T, H, N, _n.ptr(logits),
                                                     _n.ptr(workspace), int(ws_bytes), _n.stream()),
                     "om_router_gate_logits_split")
        else:
            _n.check(lib.om_router_gate_logits(_n.ptr(x), _n.ptr(weight), T, H, N, _n.ptr(logits),
                                               _n.stream()), "om_router_gate_logits")
        ctx.save_for_backward(x, weight)
        ctx.set_materialize_grads(False)
        return logits, x.view_as(x)

    @staticmethod
    def backward(ctx, dlogits, x_grad):
        x, weight = ctx.saved_tensors
        if dlogits is None:
            return x_grad, None
        return _gate_backward(x, weight, dlogits, ctx.needs_input_grad, other_grad=x_grad)


class GateLogitsF32Function(torch.autograd.Function):
    """logits = x @ weight.T for a float32 gate (om_router_gate_logits_f32) with both backward
    products (om_router_gate_dgrad_f32, om_router_gate_wgrad_f32): the float32 module's gate without
    a library GEMM."""

    @staticmethod
    def forward(ctx, x, weight):
        _n.require_cuda_contiguous(x, weight)
        T, (N, H) = x.shape[0], weight.shape
        logits = torch.empty((T, N), dtype=torch.float32, device=x.device)
        _n.check(_n.lib().om_router_gate_logits_f32(_n.ptr(x), _n.ptr(weight), T, H, N, _n.ptr(logits),
                                                    _n.stream()), "om_router_gate_logits_f32")
        ctx.save_for_backward(x, weight)
        return logits

    @staticmethod
    def backward(ctx, dlogits):
        x, weight = ctx.saved_tensors
        T, (N, H) = x.shape[0], weight.shape
        dlogits = dlogits.to(torch.float32).contiguous()
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = torch.empty_like(x)
            _n.check(_n.lib().om_router_gate_dgrad_f32(_n.ptr(dlogits), _n.ptr(weight), T, H, N, _n.ptr(dx),
                                                       _n.stream()), "om_router_gate_dgrad_f32")
        if ctx.needs_input_grad[1]:
            dw = torch.empty_like(weight)
            _n.check(_n.lib().om_router_gate_wgrad_f32(_n.ptr(x), _n.ptr(dlogits), T, H, N, _n.ptr(dw),
                                                       _n.stream()), "om_router_gate_wgrad_f32")
        return dx, dw


def fp32_logits_with_passthrough(x, weight):
    """(router logits in float32, x) from 2-D x [T,H] and weight [N,H] (the gate's nn.Linear weight).
    bf16 operands go through the gate kernels (at most 256 experts, H a multiple of 8; anything
    else raises), and the returned x is GateLogitsFunction's pass-through; a float32 module's gate
    runs on the plain float32 gate kernels (GateLogitsF32Function) and x comes back as it is."""
    if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
        _n.require_cuda_contiguous(x.contiguous(), weight.contiguous())
        # (the forward and the two backward kernels take the same shapes, so a shape that passes here
        # passes in backward)
        _require_gate_shape(weight, 8, "gate projection")
        return GateLogitsFunction.apply(x.contiguous(), weight.contiguous())
    if x.dtype == torch.float32 and weight.dtype == torch.float32:
        return GateLogitsF32Function.apply(x.contiguous(), weight.contiguous()), x
    raise TypeError(f"router gate: activations and weight must both be bfloat16 or both float32 "
                    f"(got {x.dtype}, {weight.dtype})")


def fp32_logits(x, weight):
    """Router logits in float32 (see fp32_logits_with_passthrough)."""
    return fp32_logits_with_passthrough(x, weight)[0]


def gate_logits(x, gate):
    """router_logits = gate(x) in the module's dtype (reference moe.py:456,
    modeling_olmoe.py:284) for 2-D x.  A bf16 gate runs on the gate kernels: the fp32-accumulated
    logits rounded once to bf16, which is what a bf16 linear layer returns (up to the order of the
    fp32 sum).  A float32 module's gate runs on the plain float32 gate kernels."""
    return gate_logits_with_passthrough(x, gate)[0]


def gate_logits_with_passthrough(x, gate):
    """(gate_logits(x, gate), x), the second being the gate kernels' pass-through of x for a bf16
    gate (see fp32_logits_with_passthrough) and x itself otherwise."""
    if x.dtype == torch.bfloat16 and gate.weight.dtype == torch.bfloat16:
        logits, x = fp32_logits_with_passthrough(x, gate.weight)
        return logits.to(torch.bfloat16), x
    if x.dtype == torch.float32 and gate.weight.dtype == torch.float32 and x.is_cuda and gate.bias is None:
        return fp32_logits(x, gate.weight), x
    return gate(x), x


class GateSoftmaxTopkFunction(torch.autograd.Function):
    """The OLMoE router in one launch (om_router_gate_softmax_topk): gate projection with fp32
    logits, softmax, top-K, optional renormalisation.  Returns (routing_weights, selected_experts,
    router_logits fp32, hidden_states); reference moe.py:456 and :467-471.

    The fourth output is the input itself.  A caller that feeds the experts from it (instead of from
    the tensor it passed in) makes the experts' input gradient arrive here, where the gate's own
    input gradient is added to it inside om_router_gate_dgrad: one pass over [T,H] instead of a
    matmul output plus autograd's accumulation kernel."""

    @staticmethod
    def forward(ctx, x, weight, top_k, norm_topk_prob, out_dtype):
        T, (N, H) = x.shape[0], weight.shape
        dev = x.device
        logits = torch.empty((T, N), dtype=torch.float32, device=dev)
        weights = torch.empty((T, top_k), dtype=out_dtype, device=dev)
        experts = torch.empty((T, top_k), dtype=torch.int64, device=dev)
        _n.check(_n.lib().om_router_gate_softmax_topk(
            _n.ptr(x), _n.ptr(weight), T, H, N, top_k, int(bool(norm_topk_prob)), _n.ptr(logits),
            _n.ptr(weights), _n.dtype_code(weights), _n.ptr(experts), _n.stream()),
            "om_router_gate_softmax_topk")
        ctx.save_for_backward(x, weight, logits, experts)
        ctx.norm_topk_prob = bool(norm_topk_prob)
        ctx.mark_non_differentiable(experts)
        # an output nobody differentiates (the logits without an auxiliary loss) arrives as None in
        # backward instead of a tensor of zeros that would have to be filled and added
        ctx.set_materialize_grads(False)
        return weights, experts, logits, x.view_as(x)

    @staticmethod
    def backward(ctx, weights_grad, _experts_grad, logits_grad, x_grad):
        x, weight, logits, experts = ctx.saved_tensors
        T, N = logits.shape
        K = experts.shape[1]
        if weights_grad is None and logits_grad is None:
            return x_grad, None, None, None, None
        if weights_grad is None:
            dlogits = logits_grad.to(torch.float32).contiguous()
        else:
            weights_grad = weights_grad.contiguous()
            dlogits = torch.empty_like(logits)
            _n.check(_n.lib().om_route_softmax_topk_bwd(
                _n.ptr(logits), _n.OM_F32, _n.ptr(experts), _n.ptr(weights_grad),
                _n.dtype_code(weights_grad), T, N, K, int(ctx.norm_topk_prob), _n.ptr(dlogits),
                _n.stream()), "om_route_softmax_topk_bwd")
            if logits_grad is not None:
                dlogits = dlogits + logits_grad
        dx, dw = _gate_backward(x, weight, dlogits, ctx.needs_input_grad, other_grad=x_grad)
        return dx, dw, None, None, None


class SoftmaxTopkRouterFunction(torch.autograd.Function):
    """routing_weights, selected_experts = topk(softmax_fp32(logits), K) [/ sum] -> out dtype.

    Reference moe.py:467-471.  Selection order is (probability desc, expert index asc)."""

    @staticmethod
    def forward(ctx, router_logits, top_k, norm_topk_prob, out_dtype):
        _n.require_cuda_contiguous(router_logits)
        T, N = router_logits.shape
        weights = torch.empty((T, top_k), dtype=out_dtype, device=router_logits.device)
        experts = torch.empty((T, top_k), dtype=torch.int64, device=router_logits.device)
        _n.check(_n.lib().om_route_softmax_topk(
            _n.ptr(router_logits), _n.dtype_code(router_logits), T, N, top_k, int(bool(norm_topk_prob)),
            _n.ptr(weights), _n.dtype_code(weights), _n.ptr(experts), _n.stream()),
            "om_route_softmax_topk")
        ctx.save_for_backward(router_logits, experts)
        ctx.norm_topk_prob = bool(norm_topk_prob)
        ctx.mark_non_differentiable(experts)
        return weights, experts

    @staticmethod
    def backward(ctx, weights_grad, _experts_grad):
        router_logits, experts = ctx.saved_tensors
        T, N = router_logits.shape
        K = experts.shape[1]
        weights_grad = weights_grad.contiguous()
        dlogits = torch.empty_like(router_logits)
        _n.check(_n.lib().om_route_softmax_topk_bwd(
            _n.ptr(router_logits), _n.dtype_code(router_logits), _n.ptr(experts), _n.ptr(weights_grad),
            _n.dtype_code(weights_grad), T, N, K, int(ctx.norm_topk_prob), _n.ptr(dlogits),
            _n.stream()), "om_route_softmax_topk_bwd")
        return dlogits, None, None, None


# ----------------------------------------------------------------------------------------------
# Index construction (K1 + K2 + K3)
# ----------------------------------------------------------------------------------------------
def build_token_permutation(selected_experts, expert_start_idx, expert_end_idx):
    """Stable counting sort of the (token, k) pairs routed to [expert_start_idx, expert_end_idx).

    Returns device int32 tensors (cum_token_counts [NR+1], cum_expert_counts_ep [T+1],
    input_indices, output_indices, selected_experts_indices) — the last three sized T*K; only
    the first cum_token_counts[-1] entries are meaningful.  Same values as the reference's
    K1 -> cumsum -> K3 sequence (moe.py:499-554).  Nothing is copied to the host."""
    _n.require_cuda_contiguous(selected_experts)
    T, K = selected_experts.shape
    NR = expert_end_idx - expert_start_idx
    dev = selected_experts.device
    i32 = dict(dtype=torch.int32, device=dev)
    cum_token_counts = torch.empty(NR + 1, **i32)
    cum_expert_counts_ep = torch.empty(T + 1, **i32)
    input_indices = torch.empty(T * K, **i32)
    output_indices = torch.empty(T * K, **i32)
    selected_experts_indices = torch.empty(T * K, **i32)
    ws_bytes = _n.lib().om_moe_sort_workspace_bytes(T, K, NR)
    workspace = torch.empty(max(ws_bytes // 4, 1), **i32)
    _n.check(_n.lib().om_moe_sort(
        _n.ptr(selected_experts), _n.index_code(selected_experts), T, K, int(expert_start_idx),
        int(expert_end_idx), _n.ptr(cum_token_counts), _n.ptr(cum_expert_counts_ep),
        _n.ptr(input_indices), _n.ptr(output_indices), _n.ptr(selected_experts_indices),
        _n.ptr(workspace), ws_bytes, _n.stream()), "om_moe_sort")
    return cum_token_counts, cum_expert_counts_ep, input_indices, output_indices, selected_experts_indices


# ----------------------------------------------------------------------------------------------
# Weight gradients accumulated in place
# ----------------------------------------------------------------------------------------------
# The reference trains with every p.grad a view of the optimizer's flat gradient buffer
# (optimus/optimizers.py:105-111), zeroed in place (:117-118) and accumulated into over the
# micro-batches of a step (dist_train.py:154), so autograd finishes each weight-gradient GEMM with an
# elementwise `p.grad += dW` over the whole weight.  When a weight's .grad is such a live view the
# backward functions below let the GEMM's epilogue do that sum (the *_accumulate entry points: the
# same bits) and hand autograd None for the weight.  Set to False to always return fresh gradients.
accumulate_weight_grads_in_place = True


def _live_grad(param):
    """param.grad if the weight-gradient kernels may add into it in place: a leaf parameter whose
    gradient already exists as a dense view of a larger buffer, same dtype and shape, with no hooks
    that would have to see the incoming gradient; else None."""
    if not accumulate_weight_grads_in_place or torch.is_grad_enabled():
        return None                     # (grad mode is on in backward only under create_graph)
    if not (isinstance(param, torch.Tensor) and param.is_leaf and param.requires_grad):
        return None
    grad = param.grad
    if grad is None or not grad._is_view() or grad.dtype != param.dtype or grad.shape != param.shape \
            or not grad.is_cuda or not grad.is_contiguous() or grad.requires_grad:
        return None
    if param._backward_hooks or getattr(param, "_post_accumulate_grad_hooks", None):
        return None
    return grad


def _grad_sink(leaves):
    """[G, out, in] tensor over the live gradient buffer(s) of an expert weight, or None.  `leaves`
    is the parameter itself ([G, out, in], or [out, in] for a single MLP) or the list of the G
    per-expert [out, in] parameters, whose gradients must then lie at one constant pitch inside one
    buffer (true when they are views of a flat gradient buffer in parameter order)."""
    if isinstance(leaves, (list, tuple)):
        grads = [_live_grad(w) for w in leaves]
        if any(g is None for g in grads):
            return None
        try:
            return _strided_expert_view(grads)
        except _n.NativeLibraryError:
            return None
    grad = _live_grad(leaves)
    if grad is not None and grad.dim() == 2:
        grad = grad.unsqueeze(0)
    return grad


def _weight_grad_out(sink, shape, like):
    """-> (tensor the weight-gradient GEMM writes, its expert pitch argument, accumulate flag)."""
    if sink is not None:
        return sink, _expert_stride(sink), True
    return torch.empty(shape, dtype=like.dtype, device=like.device), 0, False


# ----------------------------------------------------------------------------------------------
# Grouped GEMM functions
# ----------------------------------------------------------------------------------------------
class GroupedGemmFunction(torch.autograd.Function):
    """out[s:e] = in[s:e] @ W[g].T per expert segment (reference moe.py:163-215).

    `max_tokens_per_expert` and `use_triton_path` exist for signature parity and are ignored:
    the kernel sizes its grid from the row count and reads the offsets on the device."""

    @staticmethod
    def forward(ctx, input, merged_weight, cum_token_counts, max_tokens_per_expert=None,
                use_triton_path=False):
        _gemm_dtype(input, merged_weight)
        _n.require_cuda_contiguous(input)
        num_tokens = input.shape[0]
        num_experts, ofm, ifm = merged_weight.shape
        cum = _device_counts(cum_token_counts, input.device)
        output = torch.empty((num_tokens, ofm), dtype=input.dtype, device=input.device)
        _grouped_gemm("fwd", input, merged_weight, output, cum, num_tokens, num_experts, ofm, ifm,
                      _expert_stride(merged_weight))
        ctx.save_for_backward(input, merged_weight, cum)
        return output

    @staticmethod
    def backward(ctx, output_grad):
        input, merged_weight, cum = ctx.saved_tensors
        output_grad = output_grad.contiguous()
        num_experts, ofm, ifm = merged_weight.shape
        rows = input.shape[0]
        input_grad = torch.empty_like(input)
        weight_grad, pitch, acc = _weight_grad_out(_grad_sink(merged_weight), (num_experts, ofm, ifm),
                                                   merged_weight)
        _grouped_gemm("dgrad", output_grad, merged_weight, input_grad, cum, rows, num_experts, ofm, ifm,
                      _expert_stride(merged_weight))
        _grouped_gemm("wgrad", output_grad, input, weight_grad, cum, rows, num_experts, ofm, ifm, pitch,
                      accumulate=acc)
        return input_grad, (None if acc else weight_grad), None, None, None


def _merged_mlp_forward(x, w_gate, w_up, w_down, cum_token_counts, x_rows=None):
    """-> (y, cum, g, u, h).  Fused gate+up+SwiGLU launch, then the down projection.  With
    `x_rows` (int32 [rows]) the MLP input is x[x_rows] without that matrix being built."""
    if _gemm_dtype(x, w_gate, w_up, w_down) == torch.float32:
        return _merged_mlp_forward_f32(x, w_gate, w_up, w_down, cum_token_counts, x_rows)
    _n.require_cuda_contiguous(x, x_rows)
    rows, H = x.shape
    if x_rows is not None:
        rows = x_rows.shape[0]
    G, I, _ = w_gate.shape
    cum = _device_counts(cum_token_counts, x.device)
    g = torch.empty((rows, I), dtype=x.dtype, device=x.device)
    u = torch.empty_like(g)
    h = torch.empty_like(g)
    y = torch.empty((rows, H), dtype=x.dtype, device=x.device)
    lib = _n.lib()
    sgu = _expert_stride(w_gate)
    if _expert_stride(w_up) != sgu:
        raise _n.NativeLibraryError("gate and up expert weights must share one expert pitch")
    with record_pcl_function("1moeblock--7gmlp_fwd"):
        if x_rows is not None and rows > 0:
            _n.check(lib.om_merged_mlp_gate_up_fwd_gathered(
                _n.ptr(x), _n.ptr(x_rows), x.shape[0], _n.ptr(w_gate), _n.ptr(w_up), _n.ptr(g),
                _n.ptr(u), _n.ptr(h), _n.ptr(cum), rows, G, I, H, sgu, _n.stream()),
                "om_merged_mlp_gate_up_fwd_gathered")
        else:
            _n.check(lib.om_merged_mlp_gate_up_fwd(
                _n.ptr(x), _n.ptr(w_gate), _n.ptr(w_up), _n.ptr(g), _n.ptr(u), _n.ptr(h), _n.ptr(cum),
                rows, G, I, H, sgu, _n.stream()), "om_merged_mlp_gate_up_fwd")
        _n.check(lib.om_grouped_gemm_fwd(
            _n.ptr(h), _n.ptr(w_down), _n.ptr(y), _n.ptr(cum), rows, G, H, I,
            _expert_stride(w_down), _n.stream()), "om_grouped_gemm_fwd")
    return y, cum, g, u, h


def _gathered_rows(x, x_rows):
    if x_rows is None:
        return x
    out = torch.empty((x_rows.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    pcl_xpu_customops.index_gather(x, x_rows, out)
    return out


def _merged_mlp_forward_f32(x, w_gate, w_up, w_down, cum_token_counts, x_rows=None):
    """float32 modules: the reference's own sequence (moe.py:396-405), three grouped GEMMs and the
    SwiGLU glue kernel, on the plain fp32 kernels; nothing is fused."""
    _n.require_cuda_contiguous(x, x_rows)
    xs = _gathered_rows(x, x_rows)
    rows, H = xs.shape
    G, I, _ = w_gate.shape
    cum = _device_counts(cum_token_counts, x.device)
    g = torch.empty((rows, I), dtype=x.dtype, device=x.device)
    u = torch.empty_like(g)
    h = torch.empty_like(g)
    y = torch.empty((rows, H), dtype=x.dtype, device=x.device)
    with record_pcl_function("1moeblock--7gmlp_fwd"):
        _grouped_gemm("fwd", xs, w_gate, g, cum, rows, G, I, H, _expert_stride(w_gate))
        _grouped_gemm("fwd", xs, w_up, u, cum, rows, G, I, H, _expert_stride(w_up))
        if rows:
            _n.check(_n.lib().om_swiglu_fwd(_n.ptr(g), _n.ptr(u), _n.ptr(h), rows * I, _n.OM_F32, _n.stream()),
                     "om_swiglu_fwd")
        _grouped_gemm("fwd", h, w_down, y, cum, rows, G, H, I, _expert_stride(w_down))
    return y, cum, g, u, h


def _merged_mlp_backward_f32(dy, x, w_gate, w_up, w_down, cum, g, u, h, x_rows=None,
                             sinks=(None, None, None)):
    dy = dy.contiguous()
    xs = _gathered_rows(x, x_rows)
    rows, H = dy.shape
    G, I, _ = w_gate.shape
    new = lambda *shape: torch.empty(shape, dtype=x.dtype, device=x.device)
    dh, dg, du, dx, dx2 = new(rows, I), new(rows, I), new(rows, I), new(rows, H), new(rows, H)
    (dw_gate, sg, ag), (dw_up, su, au), (dw_down, sd, ad) = (
        _weight_grad_out(sinks[0], (G, I, H), x), _weight_grad_out(sinks[1], (G, I, H), x),
        _weight_grad_out(sinks[2], (G, H, I), x))
    with record_pcl_function("1moeblock--7gmlp_bwd"):
        _grouped_gemm("wgrad", dy, h, dw_down, cum, rows, G, H, I, sd, accumulate=ad)
        _grouped_gemm("dgrad", dy, w_down, dh, cum, rows, G, H, I, _expert_stride(w_down))
        if rows:
            _n.check(_n.lib().om_swiglu_bwd(_n.ptr(dh), _n.ptr(g), _n.ptr(u), _n.ptr(dg), _n.ptr(du), rows * I,
                                            _n.OM_F32, _n.stream()), "om_swiglu_bwd")
        _grouped_gemm("wgrad", dg, xs, dw_gate, cum, rows, G, I, H, sg, accumulate=ag)
        _grouped_gemm("wgrad", du, xs, dw_up, cum, rows, G, I, H, su, accumulate=au)
        _grouped_gemm("dgrad", dg, w_gate, dx, cum, rows, G, I, H, _expert_stride(w_gate))
        _grouped_gemm("dgrad", du, w_up, dx2, cum, rows, G, I, H, _expert_stride(w_up))
        dx += dx2
    return dx, (None if ag else dw_gate), (None if au else dw_up), (None if ad else dw_down)


def _wgrad(output_grad, input, weight_grad, cum, rows, G, N, K, pitch, accumulate, what,
           input_rows=None, output_grad_rows=None, src_rows=0):
    """One of the bf16 weight-gradient entry points: plain, with the rows of `input` or of
    `output_grad` taken through an index, each writing or (accumulate) adding into weight_grad."""
    lib, st = _n.lib(), _n.stream()
    tail = "_accumulate" if accumulate else ""
    if input_rows is not None:
        name = "om_grouped_gemm_wgrad_gathered" + tail
        rc = getattr(lib, name)(_n.ptr(output_grad), _n.ptr(input), _n.ptr(input_rows), src_rows,
                                _n.ptr(weight_grad), _n.ptr(cum), rows, G, N, K, pitch, st)
    elif output_grad_rows is not None:
        name = "om_grouped_gemm_wgrad_gathered_out" + tail
        rc = getattr(lib, name)(_n.ptr(output_grad), _n.ptr(output_grad_rows), src_rows, _n.ptr(input),
                                _n.ptr(weight_grad), _n.ptr(cum), rows, G, N, K, pitch, st)
    else:
        name = "om_grouped_gemm_wgrad" + tail
        rc = getattr(lib, name)(_n.ptr(output_grad), _n.ptr(input), _n.ptr(weight_grad), _n.ptr(cum), rows,
                                G, N, K, pitch, st)
    _n.check(rc, f"{name}({what})")


def _merged_mlp_backward(dy, x, w_gate, w_up, w_down, cum, g, u, h, x_rows=None, sinks=(None, None, None)):
    """-> (dx, dw_gate [G,I,H], dw_up [G,I,H], dw_down [G,H,I]).  With `x_rows` the MLP input was
    x[x_rows]; dx is then the gradient of that gathered matrix.  `sinks` (gate, up, down): a weight
    whose entry is a tensor gets its gradient added into that tensor by the GEMM and None returned;
    the others get a freshly allocated gradient."""
    if x.dtype == torch.float32:
        return _merged_mlp_backward_f32(dy, x, w_gate, w_up, w_down, cum, g, u, h, x_rows, sinks)
    dy = dy.contiguous()
    rows, H = dy.shape
    G, I, _ = w_gate.shape
    lib = _n.lib()
    st = _n.stream()
    dg = torch.empty_like(g)
    du = torch.empty_like(u)
    dx = torch.empty((rows, H), dtype=x.dtype, device=x.device)
    (dw_gate, sg, ag), (dw_up, su, au), (dw_down, sd, ad) = (
        _weight_grad_out(sinks[0], (G, I, H), x), _weight_grad_out(sinks[1], (G, I, H), x),
        _weight_grad_out(sinks[2], (G, H, I), x))
    with record_pcl_function("1moeblock--7gmlp_bwd"):
        _wgrad(dy, h, dw_down, cum, rows, G, H, I, sd, ad, "down")
        _n.check(lib.om_merged_mlp_down_dgrad(_n.ptr(dy), _n.ptr(w_down), _n.ptr(g), _n.ptr(u),
                                              _n.ptr(dg), _n.ptr(du), _n.ptr(cum), rows, G, I, H,
                                              _expert_stride(w_down), st), "om_merged_mlp_down_dgrad")
        gathered = dict(input_rows=x_rows, src_rows=x.shape[0]) if (x_rows is not None and rows > 0) else {}
        _wgrad(dg, x, dw_gate, cum, rows, G, I, H, sg, ag, "gate", **gathered)
        _wgrad(du, x, dw_up, cum, rows, G, I, H, su, au, "up", **gathered)
        _n.check(lib.om_merged_mlp_gate_up_dgrad(_n.ptr(dg), _n.ptr(du), _n.ptr(w_gate),
                                                 _n.ptr(w_up), _n.ptr(dx), _n.ptr(cum), rows, G,
                                                 I, H, _expert_stride(w_gate), st),
                 "om_merged_mlp_gate_up_dgrad")
    return dx, (None if ag else dw_gate), (None if au else dw_up), (None if ad else dw_down)


class MergedMLPFunction(torch.autograd.Function):
    """y = (silu(x Wg^T) * (x Wu^T)) Wd^T per expert segment, with the fused kernels:
    gate+up+SwiGLU in one launch forward; backward = down dgrad fused with the SwiGLU backward,
    one dual-operand dgrad for dx, and three weight-gradient GEMMs.

    Same mathematics as the three GroupedGemmFunction calls and two elementwise ops of the
    reference's MergedMLP.forward (moe.py:396-405) under autograd; g and u are kept in bf16 for
    the backward like the reference keeps output_gproj / output_uproj."""

    @staticmethod
    def forward(ctx, x, w_gate, w_up, w_down, cum_token_counts):
        # a single MLP may hand its three [out, in] weights over as they are
        ctx.leaves = (w_gate, w_up, w_down)
        ctx.single = w_gate.dim() == 2
        if ctx.single:
            w_gate, w_up, w_down = w_gate.unsqueeze(0), w_up.unsqueeze(0), w_down.unsqueeze(0)
        y, cum, g, u, h = _merged_mlp_forward(x, w_gate, w_up, w_down, cum_token_counts)
        ctx.save_for_backward(x, w_gate, w_up, w_down, cum, g, u, h)
        return y

    @staticmethod
    def backward(ctx, dy):
        sinks = tuple(_grad_sink(w) for w in ctx.leaves)
        dx, *dws = _merged_mlp_backward(dy, *ctx.saved_tensors, sinks=sinks)
        if ctx.single:
            dws = [None if dw is None else dw[0] for dw in dws]
        return (dx, *dws, None)


class GatheredMergedMLPFunction(torch.autograd.Function):
    """PrepareInputForGroupGemmFunction followed by MergedMLPFunction (reference moe.py:217-282 and
    :396-405) without the gathered copy of the activations: the gate/up forward GEMM and the two
    gate/up weight-gradient GEMMs read hidden_states through input_indices.  Bit-identical to the
    two functions in sequence; backward ends with the same per-token reduction of the routed rows'
    gradients (shuffle_sub_matrix_reduce)."""

    @staticmethod
    def forward(ctx, hidden_states, input_indices, cum_expert_counts_ep, output_indices, w_gate, w_up,
                w_down, cum_token_counts):
        hidden_states = hidden_states.contiguous()
        y, cum, g, u, h = _merged_mlp_forward(hidden_states, w_gate, w_up, w_down, cum_token_counts,
                                              x_rows=input_indices)
        ctx.save_for_backward(hidden_states, input_indices, cum_expert_counts_ep, output_indices, w_gate,
                              w_up, w_down, cum, g, u, h)
        return y

    @staticmethod
    def backward(ctx, dy):
        (hidden_states, input_indices, cum_expert_counts_ep, output_indices, w_gate, w_up, w_down, cum,
         g, u, h) = ctx.saved_tensors
        sinks = tuple(_grad_sink(w) for w in (w_gate, w_up, w_down))
        dx_rows, dw_gate, dw_up, dw_down = _merged_mlp_backward(dy, hidden_states, w_gate, w_up, w_down,
                                                                cum, g, u, h, x_rows=input_indices,
                                                                sinks=sinks)
        with record_pcl_function("1moeblock--6gmlp_input_prep_bwd"):
            hidden_states_grad = torch.empty_like(hidden_states)
            pcl_xpu_customops.shuffle_sub_matrix_reduce(dx_rows, cum_expert_counts_ep, output_indices,
                                                        hidden_states_grad)
        return hidden_states_grad, None, None, None, dw_gate, dw_up, dw_down, None


def _per_expert_leaves(weight_tuple):
    """(gate, up, down) lists of the per-expert parameters of a (gate_0, up_0, down_0, gate_1, ...)
    tuple."""
    N = len(weight_tuple) // 3
    return tuple([weight_tuple[3 * n + j] for n in range(N)] for j in range(3))


def _per_expert_grads(dwg, dwu, dwd, G):
    """Gradients in the (gate_0, up_0, down_0, gate_1, ...) order of the inputs; None for a
    projection whose gradient went into its live buffer."""
    flat = []
    for n in range(G):
        flat += [None if dw is None else dw[n] for dw in (dwg, dwu, dwd)]
    return flat


class GroupMLPFunction(torch.autograd.Function):
    """Un-merged layout of the reference (moe.py:43-161): weights arrive as 3*N separate
    [out, in] tensors (gate_0, up_0, down_0, gate_1, ...).  They must sit at one constant pitch
    inside a single buffer (true for parameters re-pointed into MixedPrecisionAdamW.flat_param and
    after pack_expert_weights); the same fused kernels then run on strided views, no copies."""

    @staticmethod
    def forward(ctx, input, cum_token_counts, use_triton_path, *weight_tuple):
        ctx.leaves = _per_expert_leaves(weight_tuple)
        wg, wu, wd = [_strided_expert_view(ws) for ws in ctx.leaves]
        y, cum, g, u, h = _merged_mlp_forward(input, wg, wu, wd, cum_token_counts)
        ctx.save_for_backward(input, wg, wu, wd, cum, g, u, h)
        return y

    @staticmethod
    def backward(ctx, output_grad):
        sinks = tuple(_grad_sink(ws) for ws in ctx.leaves)
        dx, dwg, dwu, dwd = _merged_mlp_backward(output_grad, *ctx.saved_tensors, sinks=sinks)
        return (dx, None, None, *_per_expert_grads(dwg, dwu, dwd, len(ctx.leaves[0])))


class GatheredGroupMLPFunction(torch.autograd.Function):
    """GroupMLPFunction on hidden_states[input_indices] without the gathered copy (see
    GatheredMergedMLPFunction); weights as in GroupMLPFunction."""

    @staticmethod
    def forward(ctx, hidden_states, input_indices, cum_expert_counts_ep, output_indices, cum_token_counts,
                *weight_tuple):
        ctx.leaves = _per_expert_leaves(weight_tuple)
        wg, wu, wd = [_strided_expert_view(ws) for ws in ctx.leaves]
        hidden_states = hidden_states.contiguous()
        y, cum, g, u, h = _merged_mlp_forward(hidden_states, wg, wu, wd, cum_token_counts,
                                              x_rows=input_indices)
        ctx.save_for_backward(hidden_states, input_indices, cum_expert_counts_ep, output_indices, wg, wu,
                              wd, cum, g, u, h)
        return y

    @staticmethod
    def backward(ctx, output_grad):
        (hidden_states, input_indices, cum_expert_counts_ep, output_indices, wg, wu, wd, cum, g, u,
         h) = ctx.saved_tensors
        sinks = tuple(_grad_sink(ws) for ws in ctx.leaves)
        dx_rows, dwg, dwu, dwd = _merged_mlp_backward(output_grad, hidden_states, wg, wu, wd, cum, g, u, h,
                                                      x_rows=input_indices, sinks=sinks)
        with record_pcl_function("1moeblock--6gmlp_input_prep_bwd"):
            hidden_states_grad = torch.empty_like(hidden_states)
            pcl_xpu_customops.shuffle_sub_matrix_reduce(dx_rows, cum_expert_counts_ep, output_indices,
                                                        hidden_states_grad)
        return (hidden_states_grad, None, None, None, None,
                *_per_expert_grads(dwg, dwu, dwd, len(ctx.leaves[0])))


def routed_mlp_unfit_reason(hidden_states, routing_weights, w_gate, w_down):
    """None when RoutedMLPFunction's kernels take these operands (bf16 activations and expert
    weights on the GPU, fp32 or bf16 routing weights, H and I multiples of 8), else why not."""
    G, I, H = w_gate.shape
    if not (hidden_states.is_cuda and hidden_states.dim() == 2):
        return "the hidden states are not a 2-D device tensor"
    if not (hidden_states.dtype == torch.bfloat16 and w_gate.dtype == torch.bfloat16
            and w_down.dtype == torch.bfloat16):
        return f"activations / expert weights are not bfloat16 ({hidden_states.dtype}, {w_gate.dtype})"
    if routing_weights.dtype not in (torch.bfloat16, torch.float32):
        return f"routing weights are {routing_weights.dtype}"
    if H % 8 != 0 or I % 8 != 0:
        return f"hidden size {H} / ffn size {I} are not multiples of 8"
    return None


def routed_mlp_kernel_fits(hidden_states, routing_weights, w_gate, w_down):
    """True when RoutedMLPFunction's kernels take these operands."""
    return routed_mlp_unfit_reason(hidden_states, routing_weights, w_gate, w_down) is None


def _routed_mlp_forward(hidden_states, routing_weights, input_indices, cum_expert_counts_ep,
                        output_indices, selected_experts_indices, w_gate, w_up, w_down,
                        cum_token_counts, residual):
    """-> (final [T,H], cum, g, u, h, row_weights): gather, weighted SwiGLU MLP, unweighted sum."""
    _n.require_cuda_contiguous(hidden_states, routing_weights, input_indices, cum_expert_counts_ep,
                               output_indices, selected_experts_indices, residual)
    _require_bf16(hidden_states, w_gate, w_up, w_down)
    T, H = hidden_states.shape
    K = routing_weights.shape[1]
    rows = input_indices.shape[0]
    G, I, _ = w_gate.shape
    dev, dt = hidden_states.device, hidden_states.dtype
    cum = _device_counts(cum_token_counts, dev)
    lib, st = _n.lib(), _n.stream()
    sgu = _expert_stride(w_gate)
    if _expert_stride(w_up) != sgu:
        raise _n.NativeLibraryError("gate and up expert weights must share one expert pitch")
    row_weights = torch.empty((rows,), dtype=torch.float32, device=dev)
    g = torch.empty((rows, I), dtype=dt, device=dev)
    u = torch.empty_like(g)
    h = torch.empty_like(g)
    y = torch.empty((rows, H), dtype=dt, device=dev)
    final = torch.empty((T, H), dtype=dt, device=dev)
    with record_pcl_function("1moeblock--7gmlp_fwd"):
        _n.check(lib.om_moe_row_weights(
            _n.ptr(routing_weights), _n.ptr(selected_experts_indices), _n.ptr(input_indices),
            _n.ptr(output_indices), _n.ptr(row_weights), rows, K, _n.dtype_code(routing_weights), st),
            "om_moe_row_weights")
        _n.check(lib.om_merged_mlp_gate_up_fwd_weighted(
            _n.ptr(hidden_states), _n.ptr(input_indices), T, _n.ptr(w_gate), _n.ptr(w_up),
            _n.ptr(row_weights), _n.ptr(g), _n.ptr(u), _n.ptr(h), _n.ptr(cum), rows, G, I, H, sgu, st),
            "om_merged_mlp_gate_up_fwd_weighted")
        _n.check(lib.om_grouped_gemm_fwd(
            _n.ptr(h), _n.ptr(w_down), _n.ptr(y), _n.ptr(cum), rows, G, H, I, _expert_stride(w_down), st),
            "om_grouped_gemm_fwd")
    with record_pcl_function("1moeblock--8gmlp_output_reduction_fwd"):
        _n.check(lib.om_sum_ggemm_output(
            _n.ptr(y), _n.ptr(cum_expert_counts_ep), _n.ptr(output_indices), _n.ptr(residual),
            _n.ptr(final), T, H, _n.dtype_code(final), st), "om_sum_ggemm_output")
    return final, cum, g, u, h, row_weights


def _routed_mlp_backward(dfinal, hidden_states, routing_weights, input_indices, cum_expert_counts_ep,
                         output_indices, selected_experts_indices, w_gate, w_up, w_down, cum, g, u, h,
                         row_weights, sinks=(None, None, None), base=None, rows_is_bound=False):
    """-> (hidden_states_grad, routing_weights_grad, dw_gate, dw_up, dw_down); `sinks` as in
    _merged_mlp_backward.  `base` [T,H]: another gradient of the same hidden states, added to the
    result inside the per-token sum (base + cast(sum of the token's rows): autograd's bits).
    `rows_is_bound`: the index arrays are sized by an upper bound of the routed rows."""
    dfinal = dfinal.contiguous()
    T, H = hidden_states.shape
    K = routing_weights.shape[1]
    rows = input_indices.shape[0]
    G, I, _ = w_gate.shape
    dev, dt = hidden_states.device, hidden_states.dtype
    lib, st = _n.lib(), _n.stream()
    dg = torch.empty_like(g)
    du = torch.empty_like(u)
    dx_rows = torch.empty((rows, H), dtype=dt, device=dev)
    (dw_gate, sg, ag), (dw_up, su, au), (dw_down, sd, ad) = (
        _weight_grad_out(sinks[0], (G, I, H), hidden_states), _weight_grad_out(sinks[1], (G, I, H), hidden_states),
        _weight_grad_out(sinks[2], (G, H, I), hidden_states))
    # the kernel writes the entry of every routed (token, k) pair; pairs outside the expert window
    # stay zero
    if rows == routing_weights.numel() and not rows_is_bound:
        routing_weights_grad = torch.empty_like(routing_weights)
    else:
        routing_weights_grad = torch.zeros_like(routing_weights)
    hidden_states_grad = torch.empty_like(hidden_states)
    with record_pcl_function("1moeblock--7gmlp_bwd"):
        if rows > 0:
            parts = lib.om_merged_mlp_row_dot_parts(I)
            if parts < 1:
                _n.check(parts, "om_merged_mlp_row_dot_parts")
            row_dot = torch.empty((parts, rows), dtype=torch.float32, device=dev)
            _wgrad(dfinal, h, dw_down, cum, rows, G, H, I, sd, ad, "down", output_grad_rows=input_indices,
                   src_rows=T)
            _n.check(lib.om_merged_mlp_down_dgrad_weighted(
                _n.ptr(dfinal), _n.ptr(input_indices), T, _n.ptr(w_down), _n.ptr(g), _n.ptr(u),
                _n.ptr(row_weights), _n.ptr(dg), _n.ptr(du), _n.ptr(row_dot), _n.ptr(cum), rows, G, I, H,
                _expert_stride(w_down), st), "om_merged_mlp_down_dgrad_weighted")
            _n.check(lib.om_moe_row_weights_grad(
                _n.ptr(row_dot), parts, _n.ptr(selected_experts_indices), _n.ptr(input_indices),
                _n.ptr(output_indices), _n.ptr(routing_weights_grad), rows, K,
                _n.dtype_code(routing_weights_grad), st), "om_moe_row_weights_grad")
            _wgrad(dg, hidden_states, dw_gate, cum, rows, G, I, H, sg, ag, "gate", input_rows=input_indices,
                   src_rows=T)
            _wgrad(du, hidden_states, dw_up, cum, rows, G, I, H, su, au, "up", input_rows=input_indices,
                   src_rows=T)
            _n.check(lib.om_merged_mlp_gate_up_dgrad(
                _n.ptr(dg), _n.ptr(du), _n.ptr(w_gate), _n.ptr(w_up), _n.ptr(dx_rows), _n.ptr(cum), rows,
                G, I, H, _expert_stride(w_gate), st), "om_merged_mlp_gate_up_dgrad")
        else:   # nothing routed to these experts: the weight gradients are zero
            for dw, n_, k_, acc in ((dw_down, H, I, ad), (dw_gate, I, H, ag), (dw_up, I, H, au)):
                if not acc:     # (a live gradient buffer stays as it is)
                    _n.check(lib.om_grouped_gemm_wgrad(None, None, _n.ptr(dw), _n.ptr(cum), 0, G, n_, k_, 0, st),
                             "om_grouped_gemm_wgrad(empty)")
    with record_pcl_function("1moeblock--6gmlp_input_prep_bwd"):
        if base is None:
            pcl_xpu_customops.shuffle_sub_matrix_reduce(dx_rows, cum_expert_counts_ep, output_indices,
                                                        hidden_states_grad)
        else:
            _n.require_cuda_contiguous(base)
            _n.check(lib.om_sum_ggemm_output(
                _n.ptr(dx_rows), _n.ptr(cum_expert_counts_ep), _n.ptr(output_indices), _n.ptr(base),
                _n.ptr(hidden_states_grad), T, H, _n.dtype_code(hidden_states_grad), st), "om_sum_ggemm_output")
    return (hidden_states_grad, routing_weights_grad, None if ag else dw_gate, None if au else dw_up,
            None if ad else dw_down)


class RoutedMLPFunction(torch.autograd.Function):
    """The expert half of the block in one function: PrepareInputForGroupGemmFunction, the SwiGLU
    MLP of every expert and GroupGemmOutputReductionFunction (reference moe.py:217-405), with both
    row permutations and the routing weight folded into the GEMMs:

      forward   h = w[t,k] * silu(x Wg^T) * (x Wu^T) formed in the gate+up epilogue (x read through
                input_indices), y = h Wd^T, final[t] = (residual[t] +) sum of the token's rows of y;
      backward  the down projection's two backward GEMMs read dfinal through input_indices, the
                SwiGLU-backward epilogue applies w and forms the routing weights' gradient
                sum_i (dfinal Wd)[i] * silu(g)[i] * u[i]; the rest as GatheredMergedMLPFunction.

    Neither the gathered input, nor the experts' output gradient w[t,k] * dfinal[t] (both [rows, H])
    is written.  The weight commutes with the linear down projection, so this is the reference's
    mathematics; h is rounded to bf16 after the weight instead of before, so results agree with the
    separate functions to bf16 accuracy, not bit for bit.

    `weights`: (gate, up, down) as [G, I, H] / [G, H, I] tensors when n_merged is true, else the
    3*G per-expert matrices of GroupMLPFunction."""

    @staticmethod
    def forward(ctx, hidden_states, routing_weights, input_indices, cum_expert_counts_ep, output_indices,
                selected_experts_indices, cum_token_counts, residual, n_merged, *weights):
        # n_merged: True = merged weights; False = per-expert weights; "bound" forms of both say that
        # the index arrays are sized by an upper bound of the routed rows (expert_computation)
        ctx.rows_is_bound = n_merged in ("merged_bound", "per_expert_bound")
        n_merged = n_merged in (True, "merged_bound")
        if n_merged:
            wg, wu, wd = ctx.leaves = weights
        else:
            ctx.leaves = _per_expert_leaves(weights)
            wg, wu, wd = [_strided_expert_view(ws) for ws in ctx.leaves]
        hidden_states = hidden_states.contiguous()
        routing_weights = routing_weights.contiguous()
        if residual is not None:
            residual = residual.contiguous()
        final, cum, g, u, h, row_weights = _routed_mlp_forward(
            hidden_states, routing_weights, input_indices, cum_expert_counts_ep, output_indices,
            selected_experts_indices, wg, wu, wd, cum_token_counts, residual)
        ctx.save_for_backward(hidden_states, routing_weights, input_indices, cum_expert_counts_ep,
                              output_indices, selected_experts_indices, wg, wu, wd, cum, g, u, h,
                              row_weights)
        ctx.n_merged = bool(n_merged)
        ctx.has_residual = residual is not None
        return final

    @staticmethod
    def backward(ctx, dfinal):
        sinks = tuple(_grad_sink(w) for w in ctx.leaves)
        dx, drw, dwg, dwu, dwd = _routed_mlp_backward(dfinal, *ctx.saved_tensors, sinks=sinks,
                                                      rows_is_bound=ctx.rows_is_bound)
        if ctx.n_merged:
            wgrads = (dwg, dwu, dwd)
        else:
            wgrads = _per_expert_grads(dwg, dwu, dwd, len(ctx.leaves[0]))
        return (dx, drw, None, None, None, None, None, dfinal if ctx.has_residual else None, None,
                *wgrads)


class RoutedAndSharedMLPFunction(torch.autograd.Function):
    """shared_mlp(x) + the routed experts' weighted sum (reference modeling_deepseek_v3.py:265,
    `self.moe(...) + self.shared_experts(residuals)`) as one function: RoutedMLPFunction over the
    per-expert weights with the shared MLP's output as its residual.  Same kernels and bits forward
    as the two functions in sequence.  Backward runs the shared MLP first and hands its input
    gradient to the routed experts' per-token sum as the base it adds to, so the two input
    gradients meet inside a kernel (base + cast(sum): what autograd's accumulation gives) and no
    separate [T,H] addition runs.

    weights: the 3*G routed matrices in GroupMLPFunction's order, then the shared MLP's gate, up,
    down [out, in] matrices."""

    @staticmethod
    def forward(ctx, hidden_states, routing_weights, input_indices, cum_expert_counts_ep, output_indices,
                selected_experts_indices, cum_token_counts, rows_is_bound, *weights):
        routed, shared = weights[:-3], weights[-3:]
        ctx.leaves = _per_expert_leaves(routed)
        ctx.shared_leaves = shared
        ctx.rows_is_bound = bool(rows_is_bound)
        wg, wu, wd = [_strided_expert_view(ws) for ws in ctx.leaves]
        sg, su, sd = [w.unsqueeze(0) for w in shared]
        hidden_states = hidden_states.contiguous()
        routing_weights = routing_weights.contiguous()
        one = single_segment_counts(hidden_states.shape[0], hidden_states.device)
        y_shared, one, gs, us, hs = _merged_mlp_forward(hidden_states, sg, su, sd, one)
        final, cum, g, u, h, row_weights = _routed_mlp_forward(
            hidden_states, routing_weights, input_indices, cum_expert_counts_ep, output_indices,
            selected_experts_indices, wg, wu, wd, cum_token_counts, y_shared)
        ctx.save_for_backward(hidden_states, routing_weights, input_indices, cum_expert_counts_ep,
                              output_indices, selected_experts_indices, wg, wu, wd, cum, g, u, h,
                              row_weights, sg, su, sd, one, gs, us, hs)
        return final

    @staticmethod
    def backward(ctx, dfinal):
        saved = ctx.saved_tensors
        routed_saved, (sg, su, sd, one, gs, us, hs) = saved[:14], saved[14:]
        hidden_states = saved[0]
        dfinal = dfinal.contiguous()
        dx_shared, *dws_shared = _merged_mlp_backward(
            dfinal, hidden_states, sg, su, sd, one, gs, us, hs,
            sinks=tuple(_grad_sink(w) for w in ctx.shared_leaves))
        dx, drw, dwg, dwu, dwd = _routed_mlp_backward(
            dfinal, *routed_saved, sinks=tuple(_grad_sink(w) for w in ctx.leaves), base=dx_shared,
            rows_is_bound=ctx.rows_is_bound)
        dws_shared = [None if dw is None else dw[0] for dw in dws_shared]
        return (dx, drw, None, None, None, None, None, None,
                *_per_expert_grads(dwg, dwu, dwd, len(ctx.leaves[0])), *dws_shared)


def _strided_expert_view(weights):
    """[G, out, in] view over per-expert matrices that lie at a constant pitch in one storage."""
    w0 = weights[0]
    o, i = w0.shape
    G = len(weights)
    if G == 1:
        return w0.unsqueeze(0)
    esz = w0.element_size()
    pitch_bytes = weights[1].data_ptr() - w0.data_ptr()
    ok = pitch_bytes > 0 and pitch_bytes % esz == 0 and pitch_bytes >= o * i * esz
    for n, w in enumerate(weights):
        ok = ok and w.is_contiguous() and w.shape == w0.shape and w.dtype == w0.dtype \
            and w.data_ptr() == w0.data_ptr() + n * pitch_bytes \
            and w.untyped_storage().data_ptr() == w0.untyped_storage().data_ptr()
    if not ok:
        raise _n.NativeLibraryError(
            "per-expert weights must lie at a constant pitch inside one buffer (merge them with "
            "pack_expert_weights, or build the optimizer first so they alias flat_param)")
    pitch = pitch_bytes // esz
    return torch.as_strided(w0, (G, o, i), (pitch, i, 1))


def has_constant_pitch(weights):
    try:
        _strided_expert_view(weights)
        return True
    except _n.NativeLibraryError:
        return False


def pack_expert_weights(experts, names=("gate_proj", "up_proj", "down_proj")):
    """Make the [out, in] weights of a ModuleList of expert MLPs lie at a constant pitch: where
    they do not already, re-point them into one buffer per projection (p.data becomes a view,
    values kept).  Module.to()/.bfloat16() re-allocates parameters one by one, so the blocks call
    this before they hand the weights to the grouped kernels."""
    for name in names:
        ws = [getattr(e, name).weight for e in experts]
        if has_constant_pitch([w.data for w in ws]):
            continue
        buf = torch.stack([w.data for w in ws]).contiguous()
        for n, w in enumerate(ws):
            w.data = buf[n]


class PrepareInputForGroupGemmFunction(torch.autograd.Function):
    """K4: ggemm_input = hidden_states[input_indices]; backward sums each token's routed rows in
    fp32 (reference moe.py:217-282).  The four trailing flags are accepted and ignored."""

    @staticmethod
    def forward(ctx, hidden_states, input_indices, cum_expert_counts_ep, output_indices,
                use_ref_path_fwd=False, use_ref_path_bwd=False,
                use_triton_path_fwd=False, use_triton_path_bwd=False):
        num_tokens, hidden_dim = hidden_states.shape
        num_routed_tokens = input_indices.shape[0]
        with record_pcl_function("1moeblock--6gmlp_input_prep_fwd"):
            ggemm_input = torch.empty((num_routed_tokens, hidden_dim), dtype=hidden_states.dtype,
                                      device=hidden_states.device)
            pcl_xpu_customops.index_gather(hidden_states.contiguous(), input_indices, ggemm_input)
        ctx.save_for_backward(cum_expert_counts_ep, output_indices)
        ctx.num_tokens = num_tokens
        ctx.hidden_dim = hidden_dim
        return ggemm_input

    @staticmethod
    def backward(ctx, ggemm_input_grad):
        cum_expert_counts_ep, output_indices = ctx.saved_tensors
        with record_pcl_function("1moeblock--6gmlp_input_prep_bwd"):
            ggemm_input_grad = ggemm_input_grad.contiguous()
            hidden_states_grad = torch.empty((ctx.num_tokens, ctx.hidden_dim),
                                             dtype=ggemm_input_grad.dtype,
                                             device=ggemm_input_grad.device)
            pcl_xpu_customops.shuffle_sub_matrix_reduce(ggemm_input_grad, cum_expert_counts_ep,
                                                        output_indices, hidden_states_grad)
        return hidden_states_grad, None, None, None, None, None, None, None


class GroupGemmOutputReductionFunction(torch.autograd.Function):
    """K6: final[t] = sum_k w[t,k] * ggemm_output[pos(t,k)] in fp32, one rounding; backward gives
    ggemm_output_grad and routing_weights_grad (reference moe.py:284-377).  The four trailing
    flags are accepted and ignored.  routing_weights may be fp32 while activations are bf16."""

    @staticmethod
    def forward(ctx, ggemm_output, routing_weights, cum_expert_counts_ep, selected_experts_indices,
                input_indices, output_indices,
                use_ref_path_fwd=False, use_ref_path_bwd=False,
                use_triton_path_fwd=False, use_triton_path_bwd=False):
        routing_weights = routing_weights.contiguous()
        ctx.save_for_backward(ggemm_output, routing_weights, cum_expert_counts_ep,
                              selected_experts_indices, input_indices, output_indices)
        num_tokens, _ = routing_weights.shape
        hidden_dim = ggemm_output.shape[1]
        with record_pcl_function("1moeblock--8gmlp_output_reduction_fwd"):
            final_hidden_states = torch.empty((num_tokens, hidden_dim), dtype=ggemm_output.dtype,
                                              device=ggemm_output.device)
            pcl_xpu_customops.reduce_ggemm_output(ggemm_output, routing_weights, cum_expert_counts_ep,
                                                  selected_experts_indices, output_indices,
                                                  final_hidden_states, False)
        return final_hidden_states

    @staticmethod
    def backward(ctx, final_hidden_states_grad):
        (ggemm_output, routing_weights, cum_expert_counts_ep, selected_experts_indices, input_indices,
         output_indices) = ctx.saved_tensors
        final_hidden_states_grad = final_hidden_states_grad.contiguous()
        ggemm_output_grad = torch.empty_like(ggemm_output)
        # the kernel writes the entry of every routed (token, k) pair; pairs outside the expert
        # window stay zero (the reference pre-zeroes the whole tensor, moe.py:336)
        if output_indices.shape[0] == routing_weights.numel():
            routing_weights_grad = torch.empty_like(routing_weights)
        else:
            routing_weights_grad = torch.zeros_like(routing_weights)
        with record_pcl_function("1moeblock--8gmlp_output_reduction_bwd"):
            pcl_xpu_customops.reduce_ggemm_output_backward(
                final_hidden_states_grad, ggemm_output, routing_weights, cum_expert_counts_ep,
                selected_experts_indices, input_indices, output_indices, ggemm_output_grad,
                routing_weights_grad)
        return ggemm_output_grad, routing_weights_grad, None, None, None, None, None, None, None, None


class GroupGemmOutputReductionResidualFunction(torch.autograd.Function):
    """residual + GroupGemmOutputReductionFunction(...) in one pass: the combined sum is rounded to
    the activation dtype and then added to `residual` (both roundings of the two-step form).  Used
    for the decoder layer's residual connection (modeling_olmoe.py:415) and for the DeepSeek-V3
    block's routed + shared sum (modeling_deepseek_v3.py:265).  The gradient of the output goes to
    `residual` unchanged and into the combine's backward."""

    @staticmethod
    def forward(ctx, ggemm_output, routing_weights, cum_expert_counts_ep, selected_experts_indices,
                input_indices, output_indices, residual):
        routing_weights = routing_weights.contiguous()
        residual = residual.contiguous()
        ctx.save_for_backward(ggemm_output, routing_weights, cum_expert_counts_ep,
                              selected_experts_indices, input_indices, output_indices)
        with record_pcl_function("1moeblock--8gmlp_output_reduction_fwd"):
            final_hidden_states = torch.empty_like(residual)
            pcl_xpu_customops.reduce_ggemm_output_residual(
                ggemm_output, routing_weights, cum_expert_counts_ep, selected_experts_indices,
                output_indices, residual, final_hidden_states)
        return final_hidden_states

    @staticmethod
    def backward(ctx, final_hidden_states_grad):
        grads = GroupGemmOutputReductionFunction.backward(ctx, final_hidden_states_grad)
        return grads[0], grads[1], None, None, None, None, final_hidden_states_grad


# ----------------------------------------------------------------------------------------------
# Modules
# ----------------------------------------------------------------------------------------------
class MergedMLP(nn.Module):
    """All local experts' SwiGLU MLPs as three 3-D parameters (reference moe.py:379-405)."""

    def __init__(self, config):
        super(MergedMLP, self).__init__()
        self.config = config
        self.num_experts_per_rank = config.num_experts // config.expert_parallelism
        self.gate_proj_merged_weight = torch.nn.Parameter(
            torch.empty((self.num_experts_per_rank, config.intermediate_size, config.hidden_size)))
        self.up_proj_merged_weight = torch.nn.Parameter(
            torch.empty((self.num_experts_per_rank, config.intermediate_size, config.hidden_size)))
        self.down_proj_merged_weight = torch.nn.Parameter(
            torch.empty((self.num_experts_per_rank, config.hidden_size, config.intermediate_size)))

    def forward(self, input, cum_token_counts):
        return MergedMLPFunction.apply(input, self.gate_proj_merged_weight, self.up_proj_merged_weight,
                                       self.down_proj_merged_weight, cum_token_counts)

    def forward_gathered(self, hidden_states, input_indices, cum_expert_counts_ep, output_indices,
                         cum_token_counts):
        """forward(hidden_states[input_indices], cum_token_counts) with the gather folded into the
        GEMMs; the two index arrays after input_indices serve the backward's per-token reduction."""
        return GatheredMergedMLPFunction.apply(hidden_states, input_indices, cum_expert_counts_ep,
                                               output_indices, self.gate_proj_merged_weight,
                                               self.up_proj_merged_weight, self.down_proj_merged_weight,
                                               cum_token_counts)


def expert_computation(hidden_states, routing_weights, selected_experts, expert_start_idx,
                       expert_end_idx, experts_fn, num_total_experts, gathered_experts_fn=None,
                       residual=None, routed_experts_fn=None, sync_free_window=False):
    """K1..K6 for 2-D hidden_states [T,H]: permute, run `experts_fn(ggemm_input, cum_token_counts)`,
    combine.  Shared by the OLMoE and DeepSeek-V3 blocks.  With `gathered_experts_fn(hidden_states,
    input_indices, cum_expert_counts_ep, output_indices, cum_token_counts)` the experts read the
    tokens through the index and K4's gathered copy is not built.  With `residual` [T,H] the result
    is residual + combine(...), added inside the combine kernel.  `routed_experts_fn(hidden_states,
    routing_weights, input_indices, cum_expert_counts_ep, output_indices, selected_experts_indices,
    cum_token_counts, residual)` may do gather, experts and combine in one function
    (RoutedMLPFunction); it returns None when its kernels do not take the operands.

    Under an expert window the number of routed rows is only known on the device.  By default it is
    read back once, like the reference does (moe.py:520).  With `sync_free_window` and a
    `routed_experts_fn` nothing is read back: the index arrays keep their T*K entries (om_moe_sort
    marks the unused tail), the activations of the expert MLP are allocated for T*K rows, of which
    only the routed ones are computed, and the function is called with `rows_is_bound=True`.  That
    makes the step capturable in a HIP graph at the price of expert_parallelism times the
    activation memory."""
    T, K = selected_experts.shape
    with record_pcl_function("1moeblock--3index_calculation"):
        (cum_token_counts, cum_expert_counts_ep, input_indices, output_indices,
         selected_experts_indices) = build_token_permutation(selected_experts, expert_start_idx,
                                                             expert_end_idx)
    windowed = not (expert_start_idx == 0 and expert_end_idx == num_total_experts)
    if windowed and sync_free_window and routed_experts_fn is not None:
        final = routed_experts_fn(hidden_states, routing_weights, input_indices, cum_expert_counts_ep,
                                  output_indices, selected_experts_indices, cum_token_counts, residual,
                                  rows_is_bound=True)
        if final is not None:
            return final
    if not windowed:
        num_routed_tokens = T * K            # every pair is local: no host read
    else:
        num_routed_tokens = int(cum_token_counts[-1].item())   # same host read as moe.py:520
    input_indices = input_indices[:num_routed_tokens]
    output_indices = output_indices[:num_routed_tokens]
    selected_experts_indices = selected_experts_indices[:num_routed_tokens]
    if routed_experts_fn is not None:
        final = routed_experts_fn(hidden_states, routing_weights, input_indices, cum_expert_counts_ep,
                                  output_indices, selected_experts_indices, cum_token_counts, residual)
        if final is not None:
            return final
    if gathered_experts_fn is not None:
        ggemm_output = gathered_experts_fn(hidden_states, input_indices, cum_expert_counts_ep,
                                           output_indices, cum_token_counts)
    else:
        ggemm_input = PrepareInputForGroupGemmFunction.apply(hidden_states, input_indices,
                                                             cum_expert_counts_ep, output_indices)
        ggemm_output = experts_fn(ggemm_input, cum_token_counts)
    if residual is not None:
        return GroupGemmOutputReductionResidualFunction.apply(
            ggemm_output, routing_weights, cum_expert_counts_ep, selected_experts_indices, input_indices,
            output_indices, residual)
    return GroupGemmOutputReductionFunction.apply(ggemm_output, routing_weights, cum_expert_counts_ep,
                                                  selected_experts_indices, input_indices,
                                                  output_indices)


class FastOlmoeParallelSparseMoeBlock(nn.Module):
    """Reference moe.py:407-632.  forward(hidden_states [B,S,H]) ->
    (final_hidden_states [B,S,H], router_logits [B*S,N] or None).

    Limits of a bfloat16 block (a shape outside them raises, nothing falls back to a library):
    at most 256 experts in the gate; hidden size and ffn size multiples of 8."""

    def __init__(self, config, pmap=None):
        super().__init__()
        from optimus.models.olmoe.modeling_olmoe import OlmoeParallelMLP
        self.config = config
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
        if not self.config.use_merged_mlp_in_fast_moe:
            self.experts = nn.ModuleList([OlmoeParallelMLP(config) for _ in range(self.num_experts_per_rank)])
        else:
            self.experts = MergedMLP(config)

        self.use_activation_checkpointing_for_moe = False
        if config.use_activation_checkpointing:
            self.use_activation_checkpointing_for_moe = config.activation_checkpointing_level & (1 << 0)

        if getattr(config, "force_uniform_routing", False):
            raise NotImplementedError("force_uniform_routing is a debug mask of the reference "
                                      "(moe.py:459-464) and is not part of this build")
        # fp32 router logits (x.float() @ Wg.float().T) instead of model-dtype logits
        self.router_logits_fp32 = bool(getattr(config, "router_logits_fp32", False))
        # merged experts read the tokens through input_indices instead of a gathered copy
        self.fuse_input_gather = bool(getattr(config, "fuse_input_gather", True))
        # the routing weight is applied inside the expert MLP and the combine's backward is folded
        # into the down projection's backward GEMMs (RoutedMLPFunction); needs fuse_input_gather
        self.fuse_routing_weights = bool(getattr(config, "fuse_routing_weights", True))
        # under an expert window: never read the routed row count back (see expert_computation)
        self.sync_free_expert_window = bool(getattr(config, "sync_free_expert_window", False))

    def _experts_fn(self, ggemm_input, cum_token_counts):
        if isinstance(self.experts, MergedMLP):
            return self.experts(ggemm_input, cum_token_counts)
        pack_expert_weights(self.experts)   # no-op once the weights share a buffer
        mlp_params = []
        for expert in self.experts:
            mlp_params += [expert.gate_proj.weight, expert.up_proj.weight, expert.down_proj.weight]
        return GroupMLPFunction.apply(ggemm_input, cum_token_counts, False, *mlp_params)

    def _gathered_experts_fn(self, hidden_states, input_indices, cum_expert_counts_ep, output_indices,
                             cum_token_counts):
        if isinstance(self.experts, MergedMLP):
            return self.experts.forward_gathered(hidden_states, input_indices, cum_expert_counts_ep,
                                                 output_indices, cum_token_counts)
        pack_expert_weights(self.experts)
        mlp_params = []
        for expert in self.experts:
            mlp_params += [expert.gate_proj.weight, expert.up_proj.weight, expert.down_proj.weight]
        return GatheredGroupMLPFunction.apply(hidden_states, input_indices, cum_expert_counts_ep,
                                              output_indices, cum_token_counts, *mlp_params)

    def _routed_experts_fn(self, hidden_states, routing_weights, input_indices, cum_expert_counts_ep,
                           output_indices, selected_experts_indices, cum_token_counts, residual,
                           rows_is_bound=False):
        if isinstance(self.experts, MergedMLP):
            weights = (self.experts.gate_proj_merged_weight, self.experts.up_proj_merged_weight,
                       self.experts.down_proj_merged_weight)
            why = routed_mlp_unfit_reason(hidden_states, routing_weights, weights[0], weights[2])
            if why is not None:
                if hidden_states.dtype == torch.bfloat16:    # (float32 modules run unfused by design)
                    note_unfused_path("routing weight inside the expert MLP", why)
                return None
            return RoutedMLPFunction.apply(hidden_states, routing_weights, input_indices,
                                           cum_expert_counts_ep, output_indices, selected_experts_indices,
                                           cum_token_counts, residual,
                                           "merged_bound" if rows_is_bound else True, *weights)
        pack_expert_weights(self.experts)
        w0, d0 = self.experts[0].gate_proj.weight, self.experts[0].down_proj.weight
        why = routed_mlp_unfit_reason(hidden_states, routing_weights, w0.unsqueeze(0), d0.unsqueeze(0))
        if why is not None:
            if hidden_states.dtype == torch.bfloat16:    # (float32 modules run unfused by design)
                note_unfused_path("routing weight inside the expert MLP", why)
            return None
        mlp_params = []
        for expert in self.experts:
            mlp_params += [expert.gate_proj.weight, expert.up_proj.weight, expert.down_proj.weight]
        return RoutedMLPFunction.apply(hidden_states, routing_weights, input_indices, cum_expert_counts_ep,
                                       output_indices, selected_experts_indices, cum_token_counts,
                                       residual, "per_expert_bound" if rows_is_bound else False, *mlp_params)

    def forward_with_residual(self, hidden_states, residual):
        """(residual + forward(hidden_states)[0], router_logits): the decoder layer's
        `hidden_states = residual + hidden_states` after the block (modeling_olmoe.py:415) folded into
        the combine kernel; same bits as the two steps."""
        return self.forward(hidden_states, residual=residual)

    def forward(self, hidden_states, residual=None):
        batch_size, sequence_length, hidden_dim = hidden_states.shape
        flat = hidden_states.reshape(-1, hidden_dim)
        gate_unfit = gate_kernel_unfit_reason(flat, self.gate.weight) if self.router_logits_fp32 else None
        if self.router_logits_fp32 and gate_unfit is not None and flat.dtype == torch.bfloat16:
            note_unfused_path("gate projection fused with the routing", gate_unfit,
                              instead="running the projection and the routing as separate kernels (same fp32 logits)")
        if self.router_logits_fp32 and gate_unfit is None:
            # the experts read the router function's pass-through of the hidden states, so that their
            # input gradient and the gate's are added in one kernel (GateSoftmaxTopkFunction)
            routing_weights, selected_experts, router_logits, flat = GateSoftmaxTopkFunction.apply(
                flat.contiguous(), self.gate.weight, self.num_experts_per_tok, self.norm_topk_prob,
                hidden_states.dtype)
            hidden_states = flat.view(batch_size, sequence_length, hidden_dim)
        else:
            # (the experts are fed from the gate projection's pass-through here too: their input
            # gradient is then added to the gate's inside om_router_gate_dgrad)
            if self.router_logits_fp32:
                router_logits, flat = fp32_logits_with_passthrough(flat, self.gate.weight)
            else:
                router_logits, flat = gate_logits_with_passthrough(flat, self.gate)
            hidden_states = flat.view(batch_size, sequence_length, hidden_dim)
            routing_weights, selected_experts = SoftmaxTopkRouterFunction.apply(
                router_logits.contiguous(), self.num_experts_per_tok, self.norm_topk_prob,
                hidden_states.dtype)

        def expert_computation_block(hidden_states, selected_experts, routing_weights, residual=None):
            b, s, h = hidden_states.shape
            gathered = self._gathered_experts_fn if self.fuse_input_gather else None
            routed = self._routed_experts_fn if (self.fuse_input_gather and self.fuse_routing_weights) else None
            out = expert_computation(hidden_states.reshape(-1, h), routing_weights, selected_experts,
                                     self.expert_start_idx, self.expert_end_idx, self._experts_fn,
                                     self.num_experts, gathered_experts_fn=gathered,
                                     residual=None if residual is None else residual.reshape(-1, h),
                                     routed_experts_fn=routed,
                                     sync_free_window=self.sync_free_expert_window)
            return out.reshape(b, s, h)

        args = [hidden_states, selected_experts, routing_weights]
        if residual is not None:
            args.append(residual)
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
        with torch.no_grad():
            for local_expert_idx in range(self.num_experts_per_rank):
                src = module.experts[self.expert_start_idx + local_expert_idx]
                if isinstance(self.experts, MergedMLP):
                    self.experts.gate_proj_merged_weight[local_expert_idx].copy_(src.gate_proj.weight.data)
                    self.experts.up_proj_merged_weight[local_expert_idx].copy_(src.up_proj.weight.data)
                    self.experts.down_proj_merged_weight[local_expert_idx].copy_(src.down_proj.weight.data)
                else:
                    self.experts[local_expert_idx].load_state_dict(src.state_dict())


# ----------------------------------------------------------------------------------------------
# Checkpoint interchange between the merged and the per-expert weight layouts
# ----------------------------------------------------------------------------------------------
_MERGED_SUFFIX = "_merged_weight"


def merged_state_dict_to_per_expert(state_dict, expert_start_id=0):
    """Rewrites '<p>.experts.<lin>_merged_weight' [NR,out,in] entries as NR entries
    '<p>.experts.<id>.<lin>.weight' (views, no copies), id = expert_start_id + local index; all
    other entries pass through.  This is the un-merging the reference does when it converts an
    expert-parallel rank's checkpoint to per-expert keys
    (evals/convert_olmoe_om_checkpoint_to_hf.py:59-88)."""
    out = {}
    for name, tensor in state_dict.items():
        tokens = name.split(".")
        if "experts" in tokens and tokens[-1].endswith(_MERGED_SUFFIX):
            linear_key = tokens[-1][: -len(_MERGED_SUFFIX)]
            for local in range(tensor.shape[0]):
                serial = ".".join(tokens[:-1] + [str(expert_start_id + local), linear_key, "weight"])
                out[serial] = tensor[local]
        else:
            out[name] = tensor
    return out


def per_expert_state_dict_to_merged(state_dict, num_local_experts, expert_start_id=0):
    """The inverse: gathers '<p>.experts.<id>.<lin>.weight' for id in
    [expert_start_id, expert_start_id + num_local_experts) into '<p>.experts.<lin>_merged_weight'
    (one stacked tensor per projection); entries of experts outside the window are dropped, all
    other entries pass through.  Same mapping as the reference's checkpoint generator for
    use_merged_mlp_in_fast_moe (generate_parallel_model.py:136-148)."""
    out, groups = {}, {}
    for name, tensor in state_dict.items():
        tokens = name.split(".")
        if "experts" in tokens:
            i = tokens.index("experts")
            if len(tokens) == i + 4 and tokens[i + 1].isdigit() and tokens[-1] == "weight":
                local = int(tokens[i + 1]) - expert_start_id
                if 0 <= local < num_local_experts:
                    key = ".".join(tokens[: i + 1] + [tokens[i + 2] + _MERGED_SUFFIX])
                    groups.setdefault(key, {})[local] = tensor
                continue
        out[name] = tensor
    for key, parts in groups.items():
        missing = [expert_start_id + j for j in range(num_local_experts) if j not in parts]
        if missing:
            raise KeyError(f"{key}: no weights for experts {missing}")
        out[key] = torch.stack([parts[j] for j in range(num_local_experts)])
    return out

