"""optimus.optimizers — MixedPrecisionAdamW with the reference's interface
(optimus/optimizers.py:19-225) and a single-pass HIP kernel for the update.

All parameters, gradients and optimizer states live in five flat buffers: `flat_param` and
`flat_grad` in the model dtype, `flat_exp_avg`, `flat_exp_avg_sq` and `flat_fp32_master_param`
in fp32.  Every `p.data` / `p.grad` of the model is a view into the first two, so backward
writes straight into the buffer the optimizer kernel reads.
"""
import torch
from torch.optim import Optimizer

from optimus import _native as _n
from optimus.profilers import record_pcl_function


class MixedPrecisionAdamW(Optimizer):
    """
    Stores all parameters, gradients, and optimizer states into a flat buffer.
    Optimizer states include exp_avg and exp_avg_sq which are in FP32
    Master weights are stored in FP32
    ## Limitations
    1. Only one param group
    2. One GPU: num_shards must be 1 (the data-parallel all-reduce is outside this build)
    """

    def __init__(self,
                 params, model,
                 lr=0.001,
                 betas=(0.9, 0.999),
                 eps=1e-08,
                 weight_decay=0.01, warmup_steps=0,
                 dtype=torch.float32, device=None,
                 num_shards=1, shard_id=0, group=None,
                 opt_disable_delayed_grad_clipping=False,
                 opt_use_two_step_grad_clipping=False,
                 opt_use_chunked_allreduce=False,
                 profiler=None,
                 tensor_parallelism=1, tp_ind=0, tp_group=None,
                 expert_parallelism=1, ep_ind=0, ep_group=None,
                 dpep_ind=0, dpep_group=None,
                 skip_optimizer_step=False):
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay)
        super().__init__(params, defaults)

        assert device is not None
        if dtype not in (torch.float32, torch.bfloat16):
            raise TypeError("MixedPrecisionAdamW: dtype must be torch.float32 or torch.bfloat16")

        self.model = model
        self.warmup_steps = warmup_steps
        self.dtype = dtype
        self.device = device
        self.opt_disable_delayed_grad_clipping = opt_disable_delayed_grad_clipping
        self.opt_use_two_step_grad_clipping = opt_use_two_step_grad_clipping
        self.opt_use_chunked_allreduce = opt_use_chunked_allreduce
        self.profiler = profiler

        self.tensor_parallelism = tensor_parallelism
        self.tp_ind = tp_ind
        self.tp_group = tp_group

        self.expert_parallelism = expert_parallelism
        self.ep_ind = ep_ind
        self.ep_group = ep_group

        assert self.expert_parallelism == 1, "This optimizer does not support expert parallelism."
        assert self.tensor_parallelism == 1, "tensor parallelism is outside the single-GPU hot path"

        self.dpep_ind = dpep_ind
        self.dpep_group = dpep_group
        self.skip_optimizer_step = skip_optimizer_step

        self.step_id = 0

        # Sharding options (reference optimizers.py:73-76); one GPU here
        if num_shards != 1:
            raise NotImplementedError("num_shards > 1 (data-parallel all-reduce) is not part of "
                                      "the single-GPU hot path")
        self.num_shards = num_shards
        self.dp_ind = shard_id
        self.group = group

        self.param_list = [p for pg in self.param_groups for p in pg["params"]]
        assert len([pg for pg in self.param_groups]) == 1, "Only one parameter group is supported"

        self.param_sizes = [p.numel() for p in self.param_list]
        self.param_start_inds = [sum(self.param_sizes[0:i]) for i in range(len(self.param_sizes))]
        self.flat_param_size = sum(self.param_sizes)

        # Flat buffers
        self.flat_param = torch.empty(self.flat_param_size, dtype=self.dtype, device=self.device)
        self.flat_grad = torch.zeros(self.flat_param_size, dtype=self.dtype, device=self.device)
        if not self.skip_optimizer_step:
            self.flat_exp_avg = torch.zeros(self.flat_param_size, dtype=torch.float32, device=self.device)
            self.flat_exp_avg_sq = torch.zeros(self.flat_param_size, dtype=torch.float32, device=self.device)
        else:
            self.flat_exp_avg = None
            self.flat_exp_avg_sq = None

        if self.dtype != torch.float32:
            if not self.skip_optimizer_step:
                self.flat_fp32_master_param = torch.zeros(self.flat_param_size, dtype=torch.float32,
                                                          device=self.device)
            else:
                self.flat_fp32_master_param = None
        else:
            # FP32 optimizer: master param and model param share one buffer
            self.flat_fp32_master_param = self.flat_param

        # Mapping parameter into flat parameter.
        for param_id, p in enumerate(self.param_list):
            start_ind = self.param_start_inds[param_id]
            end_ind = self.param_start_inds[param_id] + self.param_sizes[param_id]
            p.data = self.flat_param[start_ind:end_ind].view_as(p.data).copy_(p.data)
            p.grad = self.flat_grad[start_ind:end_ind].view_as(p.data)
            if self.dtype != torch.float32 and (not self.skip_optimizer_step):
                self.flat_fp32_master_param[start_ind:end_ind].view_as(p.data).copy_(p.data)

    def zero_grad(self):
        self.flat_grad.zero_()

    def _grad_norm_and_clip(self):
        """Gradient norm (always) and clip to 1.0 (after warm-up), reference optimizers.py:136-160.
        Same torch.nn.utils calls as the reference, on the same parameter views."""
        clip_now = self.opt_disable_delayed_grad_clipping or (self.step_id >= self.warmup_steps)
        if clip_now:
            if not self.opt_use_two_step_grad_clipping:
                grad_norm = torch.nn.utils.clip_grad_norm_(self.model.parameters(), 1.0)
            else:
                grad_norm = torch.nn.utils.get_total_norm(
                    [p.grad for p in self.model.parameters() if p.grad is not None])
                torch.nn.utils.clip_grads_with_norm_(self.model.parameters(), 1.0, grad_norm)
        else:
            grad_norm = torch.nn.utils.get_total_norm(
                [p.grad for p in self.model.parameters() if p.grad is not None])
        return grad_norm

    def step(self, closure=None):
        with record_pcl_function("4opt-step_grad-clip"):
            grad_norm = self._grad_norm_and_clip()

        with record_pcl_function("4opt-step_compute"):
            if not self.skip_optimizer_step:
                beta1, beta2 = self.defaults["betas"]
                eps = self.defaults["eps"]
                lr = self.param_groups[0]["lr"]
                weight_decay = self.defaults["weight_decay"]
                adamw_step_(self.flat_param, self.flat_grad, self.flat_fp32_master_param,
                            self.flat_exp_avg, self.flat_exp_avg_sq, self.step_id + 1, lr, beta1,
                            beta2, eps, weight_decay)
        # Update step
        self.step_id += 1

        return grad_norm

    def state_dict(self):
        opt_state_dict = {
            "flat_exp_avg": self.flat_exp_avg,
            "flat_exp_avg_sq": self.flat_exp_avg_sq,
            "flat_fp32_master_param": self.flat_fp32_master_param,
            "step_id": self.step_id
        }
        return opt_state_dict

    def load_state_dict(self, opt_state_dict):
        self.flat_exp_avg.copy_(opt_state_dict["flat_exp_avg"].to(self.device))
        self.flat_exp_avg_sq.copy_(opt_state_dict["flat_exp_avg_sq"].to(self.device))
        self.flat_fp32_master_param.copy_(opt_state_dict["flat_fp32_master_param"].to(self.device))
        self.step_id = opt_state_dict["step_id"]


def adamw_step_(flat_param, flat_grad, flat_master, flat_exp_avg, flat_exp_avg_sq, step, lr, beta1,
                beta2, eps, weight_decay):
    """One AdamW update over flat buffers, in place (the reference's compute block,
    optimus/optimizers.py:162-205, as a single HIP pass).  `step` is 1-based (step_id + 1)."""
    _n.require_cuda_contiguous(flat_param, flat_grad, flat_master, flat_exp_avg, flat_exp_avg_sq)
    n = flat_master.numel()
    if flat_grad.numel() != n or flat_exp_avg.numel() != n or flat_exp_avg_sq.numel() != n \
            or flat_param.numel() != n:
        raise ValueError("AdamW flat buffers must have the same number of elements")
    if flat_master.dtype != torch.float32 or flat_exp_avg.dtype != torch.float32 \
            or flat_exp_avg_sq.dtype != torch.float32:
        raise TypeError("master / exp_avg / exp_avg_sq must be float32")
    if flat_param.dtype == torch.float32:
        if flat_param.data_ptr() != flat_master.data_ptr() or flat_grad.dtype != torch.float32:
            raise ValueError("float32 mode: flat_fp32_master_param must alias flat_param and "
                             "flat_grad must be float32 (reference optimizers.py:100-102)")
        code = _n.OM_F32
    elif flat_param.dtype == torch.bfloat16 and flat_grad.dtype == torch.bfloat16:
        code = _n.OM_BF16
    else:
        raise TypeError("flat_param / flat_grad must both be bfloat16 or both float32")
    _n.check(_n.lib().om_adamw_step(_n.ptr(flat_param), _n.ptr(flat_grad), _n.ptr(flat_master),
                                    _n.ptr(flat_exp_avg), _n.ptr(flat_exp_avg_sq), n, float(lr),
                                    float(beta1), float(beta2), float(eps), float(weight_decay),
                                    int(step), code, _n.stream()), "om_adamw_step")
