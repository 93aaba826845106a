"""Drop-in for the reference's native-op module `pcl_xpu_customops`.

The reference builds this name as a SYCL/pybind11 extension
(pytorch_xpu_extensions/pcl.xpu.customops/csrc/ops/sparse_moe_block.sycl:538-548) and its Python
code imports it by name (optimus/custom_ops.py:2, optimus/models/common/moe.py:234, :269, :306,
:354, :508, :543).  Here the same seven functions, with the same positional signatures, argument
meaning and in-place/return conventions, call the HIP kernels of liboptimus_mi355x.so.

Like the reference ops they trust the caller for shapes and dtypes of index tensors (int32),
assume contiguous row-major tensors, run asynchronously on the current stream and allocate
nothing.  Unlike the reference they raise (instead of misreading memory) on a dtype the kernels
do not handle, on CPU tensors and on non-contiguous tensors.
"""
from optimus import _native as _n


def index_add_op(input, output, indices):
    """output[indices[c], :] += input[c, :]; returns output (sparse_moe_block.sycl:24-54)."""
    _n.require_cuda_contiguous(input, output, indices)
    C, E = input.shape
    _n.check(_n.lib().om_index_add(_n.ptr(input), _n.ptr(output), _n.ptr(indices), C, E,
                                   _n.dtype_code(input), _n.stream()), "index_add_op")
    return output


def index_gather(input, indices, output):
    """output[o, :] = input[indices[o], :]; returns output (sparse_moe_block.sycl:75-106)."""
    _n.require_cuda_contiguous(input, output, indices)
    O, E = output.shape[0], input.shape[1]
    _n.check(_n.lib().om_index_gather(_n.ptr(input), _n.ptr(indices), _n.ptr(output), O, E,
                                      _n.dtype_code(input), _n.stream()), "index_gather")
    return output


def index_gather_op(grad_output, expert_output_grad, indices):
    """expert_output_grad[c, :] = grad_output[indices[c], :].

    optimus/custom_ops.py:15 calls this name with this argument order, but the reference's pybind
    module never exports it; it is provided so IndexAddOpFunction.backward can run."""
    return index_gather(grad_output, indices, expert_output_grad)


def compute_partial_token_counts(selected_experts, partial_token_counts, expert_counts_ep,
                                 expert_start_idx, expert_end_idx):
    """K1 (sparse_moe_block.sycl:138-173); returns partial_token_counts."""
    _n.require_cuda_contiguous(selected_experts, partial_token_counts, expert_counts_ep)
    T, K = selected_experts.shape
    TH = partial_token_counts.shape[1]
    _n.check(_n.lib().om_compute_partial_token_counts(
        _n.ptr(selected_experts), _n.index_code(selected_experts), _n.ptr(partial_token_counts),
        _n.ptr(expert_counts_ep), int(expert_start_idx), int(expert_end_idx), T, K, TH,
        _n.stream()), "compute_partial_token_counts")
    return partial_token_counts


def compute_input_and_output_indices(selected_experts, partial_cum_token_counts,
                                     input_increment_buffer, cum_expert_counts_ep,
                                     selected_experts_indices, input_indices, output_indices,
                                     expert_start_idx, expert_end_idx):
    """K3 (sparse_moe_block.sycl:217-280)."""
    _n.require_cuda_contiguous(selected_experts, partial_cum_token_counts, input_increment_buffer,
                               cum_expert_counts_ep, selected_experts_indices, input_indices,
                               output_indices)
    T, K = selected_experts.shape
    TH = input_increment_buffer.shape[1]
    _n.check(_n.lib().om_compute_input_and_output_indices(
        _n.ptr(selected_experts), _n.index_code(selected_experts), _n.ptr(partial_cum_token_counts),
        _n.ptr(input_increment_buffer), _n.ptr(cum_expert_counts_ep),
        _n.ptr(selected_experts_indices), _n.ptr(input_indices), _n.ptr(output_indices),
        int(expert_start_idx), int(expert_end_idx), T, K, TH, _n.stream()),
        "compute_input_and_output_indices")


def shuffle_sub_matrix_reduce(ggemm_input_grad, cum_expert_counts_ep, output_indices,
                              hidden_states_grad):
    """K4 backward (sparse_moe_block.sycl:505-532)."""
    _n.require_cuda_contiguous(ggemm_input_grad, cum_expert_counts_ep, output_indices,
                               hidden_states_grad)
    T, E = hidden_states_grad.shape
    _n.check(_n.lib().om_shuffle_sub_matrix_reduce(
        _n.ptr(ggemm_input_grad), _n.ptr(cum_expert_counts_ep), _n.ptr(output_indices),
        _n.ptr(hidden_states_grad), T, E, _n.dtype_code(hidden_states_grad), _n.stream()),
        "shuffle_sub_matrix_reduce")


def reduce_ggemm_output(ggemm_output, routing_weights, cum_expert_counts_ep,
                        selected_experts_indices, output_indices, final_hidden_states,
                        skip_weights_scaling=False):
    """K6 forward (sparse_moe_block.sycl:314-362)."""
    _n.require_cuda_contiguous(ggemm_output, routing_weights, cum_expert_counts_ep,
                               selected_experts_indices, output_indices, final_hidden_states)
    T, K = routing_weights.shape
    E = ggemm_output.shape[1]
    _n.check(_n.lib().om_reduce_ggemm_output(
        _n.ptr(ggemm_output), _n.ptr(routing_weights), _n.ptr(cum_expert_counts_ep),
        _n.ptr(selected_experts_indices), _n.ptr(output_indices), _n.ptr(final_hidden_states),
        T, K, E, _n.dtype_code(ggemm_output), _n.dtype_code(routing_weights),
        int(bool(skip_weights_scaling)), _n.stream()), "reduce_ggemm_output")


def reduce_ggemm_output_residual(ggemm_output, routing_weights, cum_expert_counts_ep,
                                 selected_experts_indices, output_indices, residual, final_hidden_states):
    """K6 forward with the addition that follows it folded in: final = residual + combine(...),
    the combined sum rounded to the activation dtype before the addition (not in the reference's
    module; see om_reduce_ggemm_output_residual)."""
    _n.require_cuda_contiguous(ggemm_output, routing_weights, cum_expert_counts_ep,
                               selected_experts_indices, output_indices, residual, final_hidden_states)
    T, K = routing_weights.shape
    E = ggemm_output.shape[1]
    _n.check(_n.lib().om_reduce_ggemm_output_residual(
        _n.ptr(ggemm_output), _n.ptr(routing_weights), _n.ptr(cum_expert_counts_ep),
        _n.ptr(selected_experts_indices), _n.ptr(output_indices), _n.ptr(residual),
        _n.ptr(final_hidden_states), T, K, E, _n.dtype_code(ggemm_output),
        _n.dtype_code(routing_weights), _n.stream()), "reduce_ggemm_output_residual")


def reduce_ggemm_output_backward(final_hidden_states_grad, ggemm_output, routing_weights,
                                 cum_expert_counts_ep, selected_experts_indices, input_indices,
                                 output_indices, ggemm_output_grad, routing_weights_grad):
    """K6 backward (sparse_moe_block.sycl:425-475); routing_weights_grad must be pre-zeroed."""
    _n.require_cuda_contiguous(final_hidden_states_grad, ggemm_output, routing_weights,
                               selected_experts_indices, input_indices, output_indices,
                               ggemm_output_grad, routing_weights_grad)
    RT, E = ggemm_output.shape
    K = routing_weights.shape[1]
    _n.check(_n.lib().om_reduce_ggemm_output_backward(
        _n.ptr(final_hidden_states_grad), _n.ptr(ggemm_output), _n.ptr(routing_weights),
        _n.ptr(selected_experts_indices), _n.ptr(input_indices), _n.ptr(output_indices),
        _n.ptr(ggemm_output_grad), _n.ptr(routing_weights_grad), RT, K, E,
        _n.dtype_code(ggemm_output), _n.dtype_code(routing_weights), _n.stream()),
        "reduce_ggemm_output_backward")
