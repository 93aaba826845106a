"""optimus.custom_ops — same class as the reference (optimus/custom_ops.py:4-16)."""
import torch
import pcl_xpu_customops


class IndexAddOpFunction(torch.autograd.Function):
    """final_output[indices[c], :] += expert_output[c, :] (in place), differentiable.

    Reference: optimus/custom_ops.py:4-16.  Its backward calls `index_gather_op`, which the
    reference's native module does not export; here that name exists, so backward works:
    d(expert_output)[c, :] = grad_output[indices[c], :].  The gradient of `final_output`
    is grad_output itself (the reference returns None there)."""

    @staticmethod
    def forward(ctx, expert_output, final_output, indices):
        pcl_xpu_customops.index_add_op(expert_output, final_output, indices)
        ctx.save_for_backward(indices, expert_output)
        ctx.mark_dirty(final_output)
        return final_output

    @staticmethod
    def backward(ctx, grad_output):
        indices, expert_output = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        expert_output_grad = torch.empty_like(expert_output)
        pcl_xpu_customops.index_gather_op(grad_output, expert_output_grad, indices)
        return expert_output_grad, grad_output, None
