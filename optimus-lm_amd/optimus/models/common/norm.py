"""RMSNorm of the decoder layer on the HIP kernels (om_rmsnorm_fwd / om_rmsnorm_bwd), with the
reference modules' interface (optimus/models/olmoe/modeling_olmoe.py:93-104,
optimus/models/deepseek_v3/modeling_deepseek_v3.py:29-44), plus the fused form
`h = x + residual; y = norm(h)` of the layer body (modeling_olmoe.py:402-409), which saves the
separate elementwise add and its extra pass over the activations."""
import torch
import torch.nn as nn

from optimus import _native as _n


class RMSNormFunction(torch.autograd.Function):
    """(y, h) = (weight * cast(h * rstd), x + residual); residual may be None (then h is x)."""

    @staticmethod
    def forward(ctx, x, residual, weight, eps):
        _n.require_cuda_contiguous(x, weight)
        if weight.dtype != x.dtype or (residual is not None and residual.dtype != x.dtype):
            raise TypeError("RMSNorm: x, residual and weight must share one dtype")
        E = x.shape[-1]
        rows = x.numel() // E
        out = torch.empty_like(x)
        h = torch.empty_like(x) if residual is not None else x
        rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
        if residual is not None:
            _n.require_cuda_contiguous(residual)
        _n.check(_n.lib().om_rmsnorm_fwd(
            _n.ptr(x), _n.ptr(residual), _n.ptr(weight), float(eps), _n.ptr(out),
            _n.ptr(h) if residual is not None else None, _n.ptr(rstd), rows, E, _n.dtype_code(x),
            _n.stream()), "om_rmsnorm_fwd")
        ctx.save_for_backward(h, weight, rstd)
        ctx.has_residual = residual is not None
        return out, h

    @staticmethod
    def backward(ctx, gy, gh):
        h, weight, rstd = ctx.saved_tensors
        E = h.shape[-1]
        rows = h.numel() // E
        gy = gy.contiguous()
        dx = torch.empty_like(h)
        dw = torch.empty_like(weight)
        ws_bytes = _n.lib().om_rmsnorm_bwd_workspace_bytes(rows, E)
        ws = torch.empty(max(ws_bytes, 8), dtype=torch.uint8, device=h.device)
        _n.check(_n.lib().om_rmsnorm_bwd(_n.ptr(gy), _n.ptr(h), _n.ptr(weight), _n.ptr(rstd), _n.ptr(dx),
                                         _n.ptr(dw), _n.ptr(ws), ws_bytes, rows, E, _n.dtype_code(h),
                                         _n.stream()), "om_rmsnorm_bwd")
        if gh is not None:
            dx = dx + gh          # h also feeds the next residual connection
        return dx, (dx if ctx.has_residual else None), dw, None


class ParallelRMSNorm(nn.Module):
    def __init__(self, hidden_size, eps=1e-5):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def forward(self, hidden_states):
        y, _ = RMSNormFunction.apply(hidden_states.contiguous(), None, self.weight, self.variance_epsilon)
        return y

    def forward_with_residual(self, hidden_states, residual):
        """(norm(hidden_states + residual), hidden_states + residual) in one pass."""
        return RMSNormFunction.apply(hidden_states.contiguous(), residual.contiguous(), self.weight,
                                     self.variance_epsilon)

    def set_parameters_from_full_module(self, module):
        self.load_state_dict(module.state_dict())
