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

        # Gradient-norm kernels run over flat_grad when it holds every gradient of the model
        # (the reference takes the norm over model.parameters(), optimizers.py:143-158)
        self.opt_store_clipped_grads = True   # leave flat_grad clipped after step(), as the reference does
        owned = {id(p) for p in self.param_list}
        model_params = list(self.model.parameters()) if self.model is not None else self.param_list
        if self.flat_param_size > 0 and len(model_params) == len(owned) \
                and all(id(p) in owned for p in model_params):
            self._norm_plan = GradNormPlan(self.param_start_inds, self.param_sizes, self.device)
        else:
            self._norm_plan = None

    def zero_grad(self):
        self.flat_grad.zero_()

    def _grad_norm_and_clip(self):
        """Gradient norm (always) and the clip to 1.0 (after warm-up), reference
        optimizers.py:136-160.  Returns (grad_norm, clip_coef): grad_norm is a 0-dim tensor in the
        gradient dtype like torch.nn.utils.get_total_norm gives; clip_coef is a device fp32 scalar
        for the update kernel to apply, or None when this step does not clip.  The single-step
        and two-step variants of the reference compute the same thing on one device."""
        clip_now = self.opt_disable_delayed_grad_clipping or (self.step_id >= self.warmup_steps)
        if self._norm_plan is None:
            # the model holds parameters this optimizer does not own: their gradients are not in
            # flat_grad, so take the norm over the model's list with the library calls
            grads = [p.grad for p in self.model.parameters() if p.grad is not None]
            grad_norm = torch.nn.utils.get_total_norm(grads)
            if clip_now:
                torch.nn.utils.clip_grads_with_norm_(self.model.parameters(), 1.0, grad_norm)
            return grad_norm, None
        total, coef = self._norm_plan.run(self.flat_grad, max_norm=1.0)
        return total.to(self.flat_grad.dtype), (coef if clip_now else None)

    def step(self, closure=None):
        with record_pcl_function("4opt-step_grad-clip"):
            grad_norm, clip_coef = self._grad_norm_and_clip()

        with record_pcl_function("4opt-step_compute"):
            if not self.skip_optimizer_step:
                beta1, beta2 = self.defaults["betas"]
                eps = self.defaults["eps"]
                lr = self.param_groups[0]["lr"]
                weight_decay = self.defaults["weight_decay"]
                adamw_step_(self.flat_param, self.flat_grad, self.flat_fp32_master_param,
                            self.flat_exp_avg, self.flat_exp_avg_sq, self.step_id + 1, lr, beta1,
                            beta2, eps, weight_decay, grad_scale=clip_coef,
                            store_scaled_grad=self.opt_store_clipped_grads)
            elif clip_coef is not None:
                # no update kernel to fold the clip into
                self.flat_grad.mul_(clip_coef.to(self.flat_grad.dtype))
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
                beta2, eps, weight_decay, grad_scale=None, store_scaled_grad=True):
    """One AdamW update over flat buffers, in place (the reference's compute block,
    optimus/optimizers.py:162-205, as a single HIP pass).  `step` is 1-based (step_id + 1).
    `grad_scale` (device fp32 scalar) folds the gradient clip in: the update uses
    cast(grad * grad_scale), and stores it back into flat_grad if `store_scaled_grad`."""
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
    args = (_n.ptr(flat_param), _n.ptr(flat_grad), _n.ptr(flat_master), _n.ptr(flat_exp_avg),
            _n.ptr(flat_exp_avg_sq), n, float(lr), float(beta1), float(beta2), float(eps),
            float(weight_decay), int(step), code)
    if grad_scale is None:
        _n.check(_n.lib().om_adamw_step(*args, _n.stream()), "om_adamw_step")
    else:
        _n.require_cuda_contiguous(grad_scale)
        if grad_scale.dtype != torch.float32 or grad_scale.numel() != 1:
            raise TypeError("grad_scale must be one float32 element on the device")
        _n.check(_n.lib().om_adamw_step_clipped(*args, _n.ptr(grad_scale), int(bool(store_scaled_grad)),
                                                _n.stream()), "om_adamw_step_clipped")


class GradNormPlan:
    """Chunk tables and scratch for the gradient-norm kernels over one flat gradient buffer.

    `starts[i]`, `sizes[i]` give parameter i's slice of the flat buffer (reference
    optimizers.py:86-92 `param_start_inds`, `param_sizes`).  The norm of every slice, the norm of
    those norms and the clip coefficient come out as torch.nn.utils.get_total_norm and
    clip_grads_with_norm_ compute them, including the roundings to the gradient dtype."""

    CHUNK = 1 << 16

    def __init__(self, starts, sizes, device, chunk=None):
        chunk = int(chunk or self.CHUNK)
        if len(sizes) == 0 or len(starts) != len(sizes):
            raise ValueError("GradNormPlan needs one (start, size) pair per parameter")
        begins, first, pos = [], [0], int(starts[0])
        for st, sz in zip(starts, sizes):
            st, sz = int(st), int(sz)
            if st != pos:
                raise ValueError("GradNormPlan: parameter slices must tile the flat buffer in order, "
                                 "without gaps")
            begins.append(torch.arange(st, st + sz, chunk, dtype=torch.int64))
            first.append(first[-1] + (sz + chunk - 1) // chunk)
            pos = st + sz
        table = torch.cat(begins + [torch.tensor([pos], dtype=torch.int64)])
        self.n_chunks = first[-1]
        self.n_segs = len(sizes)
        self.chunk_offsets = table.to(device)
        self.seg_first_chunk = torch.tensor(first, dtype=torch.int64).to(device)
        self.partials = torch.empty(max(self.n_chunks, 1), dtype=torch.float32, device=device)
        self.seg_norms = torch.empty(self.n_segs, dtype=torch.float32, device=device)
        self.out = torch.empty(2, dtype=torch.float32, device=device)   # total norm, clip coef

    def run(self, flat_grad, max_norm=1.0):
        """Returns (total_norm, clip_coef) as 0-dim float32 device tensors (views of one buffer
        that the next call overwrites)."""
        _n.require_cuda_contiguous(flat_grad)
        code = _n.dtype_code(flat_grad)
        lib = _n.lib()
        _n.check(lib.om_grad_sumsq(_n.ptr(flat_grad), code, _n.ptr(self.chunk_offsets), self.n_chunks,
                                   _n.ptr(self.partials), _n.stream()), "om_grad_sumsq")
        _n.check(lib.om_grad_norm_clip_coef(_n.ptr(self.partials), _n.ptr(self.seg_first_chunk),
                                            self.n_segs, code, float(max_norm), _n.ptr(self.seg_norms),
                                            _n.ptr(self.out), _n.ptr(self.out) + 4, _n.stream()),
                 "om_grad_norm_clip_coef")
        return self.out[0], self.out[1:2]
