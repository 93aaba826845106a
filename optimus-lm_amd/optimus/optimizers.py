"""optimus.optimizers — MixedPrecisionAdamW and ShardedMixedPrecisionAdamW with the reference's
interfaces (optimus/optimizers.py:19-225, :227-522) and a single-pass HIP kernel for the update.

All parameters, gradients and optimizer states live in five flat buffers: `flat_param` and
`flat_grad` in the model dtype, `flat_exp_avg`, `flat_exp_avg_sq` and `flat_fp32_master_param`
in fp32.  Every `p.data` / `p.grad` of the model is a view into the first two, so backward
writes straight into the buffer the optimizer kernel reads.
"""
import torch
from torch.optim import Optimizer

from optimus import _native as _n
from optimus.profilers import record_pcl_function


_STATE_KEYS = ("flat_exp_avg", "flat_exp_avg_sq", "flat_fp32_master_param")
_SHARD_STATE_KEYS = ("flat_exp_avg_shard", "flat_exp_avg_sq_shard", "flat_fp32_master_param_shard")
_ALLREDUCE_PART = 128 * 1024 * 1024      # elements per call of the chunked all-reduce (optimizers.py:11-17)


class ProcessGroupExchange:
    """The collectives of the optimizers' steps, made through torch.distributed exactly where the
    reference makes them (optimus/optimizers.py:120-133 unsharded; :362-375, :402, :481-494 sharded).
    Without an initialised process group `active()` is false and the step is the single-process
    one.  Tests replace the optimizer's `exchange` attribute with an in-process stand-in."""

    def active(self):
        return torch.distributed.is_available() and torch.distributed.is_initialized()

    def reduce_scatter(self, shard, full, group):
        torch.distributed.reduce_scatter_tensor(shard, full, group=group)

    def all_reduce(self, tensor, group=None):
        torch.distributed.all_reduce(tensor, group=group)

    def all_gather(self, full, shard, group):
        torch.distributed.all_gather_into_tensor(full, shard, group=group)


class MixedPrecisionAdamW(Optimizer):
    """AdamW over five flat buffers, interface of the reference class (optimus/optimizers.py:19-225).

    `flat_param` / `flat_grad` hold every parameter and gradient in the model dtype, back to back in
    `param_list` order; `flat_exp_avg`, `flat_exp_avg_sq`, `flat_fp32_master_param` are float32.  After
    construction each `p.data` and `p.grad` is a view of its slice, so backward accumulates straight
    into the buffer the update kernel reads.  In float32 mode the master weights are `flat_param`
    itself.  Constraints kept from the reference: one parameter group, `device` given, no expert
    parallelism; beyond it: no tensor parallelism, float32 or bfloat16.  With `num_shards > 1` and an
    initialised process group the gradients are all-reduced over `group` and averaged before the
    norm, where the reference does it (optimus/optimizers.py:120-133); without a process group the
    step is the single-process one.
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
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        if device is None:
            raise AssertionError("MixedPrecisionAdamW needs the device of the flat buffers")
        if dtype not in (torch.float32, torch.bfloat16):
            raise TypeError("MixedPrecisionAdamW: dtype must be torch.float32 or torch.bfloat16")
        if len(self.param_groups) != 1:
            raise AssertionError("Only one parameter group is supported")
        if expert_parallelism != 1:
            raise AssertionError("This optimizer does not support expert parallelism.")
        if tensor_parallelism != 1:
            raise AssertionError("tensor parallelism is outside the single-GPU hot path")
        # attributes the training driver and the sharded variants of the reference read
        for name, value in (("model", model), ("warmup_steps", warmup_steps), ("dtype", dtype),
                            ("device", device), ("profiler", profiler), ("group", group),
                            ("num_shards", num_shards), ("dp_ind", shard_id),
                            ("opt_disable_delayed_grad_clipping", opt_disable_delayed_grad_clipping),
                            ("opt_use_two_step_grad_clipping", opt_use_two_step_grad_clipping),
                            ("opt_use_chunked_allreduce", opt_use_chunked_allreduce),
                            ("tensor_parallelism", tensor_parallelism), ("tp_ind", tp_ind),
                            ("tp_group", tp_group), ("expert_parallelism", expert_parallelism),
                            ("ep_ind", ep_ind), ("ep_group", ep_group), ("dpep_ind", dpep_ind),
                            ("dpep_group", dpep_group), ("skip_optimizer_step", skip_optimizer_step)):
            setattr(self, name, value)
        self.step_id = 0
        self.opt_store_clipped_grads = True   # leave flat_grad clipped after step(), as the reference does
        self.exchange = ProcessGroupExchange()

        # layout: one running offset over the group's parameters
        self.param_list = list(self.param_groups[0]["params"])
        self.param_sizes, self.param_start_inds, offset = [], [], 0
        for p in self.param_list:
            self.param_start_inds.append(offset)
            self.param_sizes.append(p.numel())
            offset += p.numel()
        self.flat_param_size = offset

        def buffer(dt, zero=True):
            make = torch.zeros if zero else torch.empty
            return make(self.flat_param_size, dtype=dt, device=device)

        keep_state = not skip_optimizer_step
        self.flat_param = buffer(dtype, zero=False)
        self.flat_grad = buffer(dtype)
        self.flat_exp_avg = buffer(torch.float32) if keep_state else None
        self.flat_exp_avg_sq = buffer(torch.float32) if keep_state else None

        # move the parameters in: their values first, then re-point data and grad at the slices
        if self.param_list:
            slices = self.flat_param.split(self.param_sizes)
            grad_slices = self.flat_grad.split(self.param_sizes)
            with torch.no_grad():
                for p, dst, gdst in zip(self.param_list, slices, grad_slices):
                    dst = dst.view(p.shape)
                    dst.copy_(p.data)
                    p.data = dst
                    p.grad = gdst.view(p.shape)
        if dtype == torch.float32:
            self.flat_fp32_master_param = self.flat_param          # one buffer serves as both
        elif keep_state:
            self.flat_fp32_master_param = self.flat_param.to(torch.float32)   # exact widening, one pass
        else:
            self.flat_fp32_master_param = None

        self._norm_plan = GradNormPlan(self.param_start_inds, self.param_sizes, device) \
            if self.flat_param_size > 0 else None
        self._foreign_plans = {}

    def zero_grad(self):
        self.flat_grad.zero_()

    def _foreign_grads(self):
        """Gradients of model parameters that this optimizer does not hold in flat_grad (the
        reference takes the norm, and clips, over model.parameters(), optimizers.py:143-158)."""
        if self.model is None:
            return []
        owned = {id(p) for p in self.param_list}
        return [p.grad for p in self.model.parameters() if id(p) not in owned and p.grad is not None]

    def _grad_norm_and_clip(self):
        """Gradient norm (always) and the clip to 1.0 (after warm-up), reference
        optimizers.py:136-160.  Returns (grad_norm, clip_coef): grad_norm is a fresh 0-dim tensor in
        the gradient dtype like torch.nn.utils.get_total_norm gives; clip_coef is a device fp32
        scalar for the update kernel to apply, or None when this step does not clip.  The
        single-step and two-step variants of the reference compute the same thing on one device.
        Gradients outside flat_grad are measured by the same kernels (one extra launch per tensor)
        and scaled in place here, since no update kernel touches them."""
        clip_now = self.opt_disable_delayed_grad_clipping or (self.step_id >= self.warmup_steps)
        foreign = self._foreign_grads()
        if self._norm_plan is None and not foreign:
            zero = torch.zeros((), dtype=self.flat_grad.dtype, device=self.device)
            return zero, None
        total, coef = run_grad_norm(self._norm_plan, self.flat_grad, foreign, self._foreign_plans,
                                    max_norm=1.0)
        if clip_now:
            for g in foreign:
                scale_grad_(g, coef)
        return total.to(self.flat_grad.dtype, copy=True), (coef if clip_now else None)

    def step(self, closure=None):
        with record_pcl_function("3dp-comms-1grad_acc-block"):
            if self.num_shards > 1 and self.flat_param_size > 0 and self.exchange.active():
                parts = self.flat_grad.split(_ALLREDUCE_PART) if self.opt_use_chunked_allreduce \
                    else (self.flat_grad,)
                for part in parts:
                    self.exchange.all_reduce(part, self.group)
                self.flat_grad.div_(self.num_shards)
        with record_pcl_function("4opt-step_grad-clip"):
            grad_norm, clip_coef = self._grad_norm_and_clip()

        with record_pcl_function("4opt-step_compute"):
            if self.flat_param_size == 0:
                pass
            elif not self.skip_optimizer_step:
                group = self.param_groups[0]
                beta1, beta2 = self.defaults["betas"]
                adamw_step_(self.flat_param, self.flat_grad, self.flat_fp32_master_param,
                            self.flat_exp_avg, self.flat_exp_avg_sq, self.step_id + 1, group["lr"], beta1,
                            beta2, self.defaults["eps"], self.defaults["weight_decay"],
                            grad_scale=clip_coef, store_scaled_grad=self.opt_store_clipped_grads)
            elif clip_coef is not None:
                scale_grad_(self.flat_grad, clip_coef)   # no update kernel to fold the clip into
        self.step_id += 1
        return grad_norm

    def state_dict(self):
        state = {key: getattr(self, key) for key in _STATE_KEYS}
        state["step_id"] = self.step_id
        return state

    def load_state_dict(self, opt_state_dict):
        for key in _STATE_KEYS:
            getattr(self, key).copy_(opt_state_dict[key].to(self.device))
        self.step_id = opt_state_dict["step_id"]


class ShardedMixedPrecisionAdamW(Optimizer):
    """AdamW whose fp32 master weights and moments exist only for this rank's shard of the flat
    buffer; interface of the reference class (optimus/optimizers.py:227-522).

    `flat_param` / `flat_grad` span `num_shards * shard_size` elements in the model dtype (the
    parameters back to back, then zero padding up to a multiple of `shard_divisible_by` per shard);
    `flat_param_shard` / `flat_grad_shard` are this rank's slices and `flat_exp_avg_shard`,
    `flat_exp_avg_sq_shard`, `flat_fp32_master_param_shard` its float32 states.  One step is: gradient
    exchange (reduce-scatter, or all-reduce), the shard's norm, the all-reduced total norm, the clip
    and the AdamW update of the shard in ONE kernel pass, parameter exchange (all-gather, or
    all-reduce).  Norm, coefficient and clip decision stay on the device: the reference's
    `if clip_coef < 1.0` (:431) reads the norm back every step, here a one-thread kernel turns it into
    a multiplier (1 when nothing is to be clipped) that the update kernel applies.

    Kept from the reference: one parameter group, `device` given.  Beyond it: no expert or tensor
    parallelism (their replicated-parameter rescaling needs model hooks outside this path);
    `shard_size` a multiple of 8; in float32 mode the master shard is `flat_param_shard` itself (the
    reference keeps a second float32 copy with the same values)."""

    def __init__(self,
                 params, model,
                 lr=0.001,
                 betas=(0.9, 0.999),
                 eps=1e-08,
                 weight_decay=0.01, warmup_steps=0,
                 dtype=torch.float32, device=None,
                 num_shards=1, shard_id=0, group=None,
                 opt_disable_delayed_grad_clipping=False,
                 profiler=None,
                 tensor_parallelism=1, tp_ind=0, tp_group=None,
                 expert_parallelism=1, ep_ind=0, ep_group=None,
                 dpep_ind=0, dpep_group=None,
                 shard_divisible_by=512,
                 opt_use_chunked_allreduce=False,
                 opt_use_allreduce_for_grad_acc=False,
                 opt_use_allreduce_for_param_gather=False,
                 skip_optimizer_step=False,
                 disable_optimizer_state_checkpointing=False,
                 skip_optimizer_step_weight_update=False):
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        if device is None:
            raise AssertionError("ShardedMixedPrecisionAdamW needs the device of the flat buffers")
        if dtype not in (torch.float32, torch.bfloat16):
            raise TypeError("ShardedMixedPrecisionAdamW: dtype must be torch.float32 or torch.bfloat16")
        if len(self.param_groups) != 1:
            raise AssertionError("Only one parameter group is supported")
        if expert_parallelism != 1 or tensor_parallelism != 1:
            raise AssertionError("expert / tensor parallelism are outside the single-GPU hot path")
        if not 0 <= shard_id < num_shards:
            raise ValueError(f"shard_id {shard_id} outside [0, {num_shards})")
        self.opt_key = "shard"
        for name, value in (("model", model), ("warmup_steps", warmup_steps), ("dtype", dtype),
                            ("device", device), ("profiler", profiler),
                            ("opt_disable_delayed_grad_clipping", opt_disable_delayed_grad_clipping),
                            ("tensor_parallelism", tensor_parallelism), ("tp_ind", tp_ind),
                            ("tp_group", tp_group), ("expert_parallelism", expert_parallelism),
                            ("ep_ind", ep_ind), ("ep_group", ep_group), ("dpep_ind", dpep_ind),
                            ("dpep_group", dpep_group),
                            ("data_parallelism", num_shards), ("dp_ind", shard_id), ("dp_group", group),
                            ("shard_divisible_by", shard_divisible_by),
                            ("opt_use_chunked_allreduce", opt_use_chunked_allreduce),
                            ("opt_use_allreduce_for_grad_acc", opt_use_allreduce_for_grad_acc),
                            ("opt_use_allreduce_for_param_gather", opt_use_allreduce_for_param_gather),
                            ("skip_optimizer_step", skip_optimizer_step),
                            ("disable_optimizer_state_checkpointing", disable_optimizer_state_checkpointing),
                            ("skip_optimizer_step_weight_update", skip_optimizer_step_weight_update)):
            setattr(self, name, value)
        self.step_id = 0
        self.dump_weight_gradients = False     # a debugging switch the reference's trainer sets
        self.exchange = ProcessGroupExchange()

        self.param_list = list(self.param_groups[0]["params"])
        self.param_sizes, self.param_start_inds, offset = [], [], 0
        for p in self.param_list:
            self.param_start_inds.append(offset)
            self.param_sizes.append(p.numel())
            offset += p.numel()
        self.flat_param_size = offset

        # every shard holds a whole number of `shard_divisible_by` blocks (optimizers.py:297-298)
        block = num_shards * shard_divisible_by
        self.shard_size = (offset + block - 1) // block * shard_divisible_by
        self.flat_buffer_size = num_shards * self.shard_size
        if self.shard_size % 8:
            raise ValueError("shard_size must be a multiple of 8 elements (16-byte aligned shard views); "
                             f"got {self.shard_size} from shard_divisible_by={shard_divisible_by}")

        self.flat_param = torch.zeros(self.flat_buffer_size, dtype=dtype, device=device)
        self.flat_grad = torch.zeros(self.flat_buffer_size, dtype=dtype, device=device)
        lo = shard_id * self.shard_size
        self.flat_param_shard = self.flat_param.narrow(0, lo, self.shard_size)
        self.flat_grad_shard = self.flat_grad.narrow(0, lo, self.shard_size)

        if self.param_list:
            pad = [self.flat_buffer_size - offset] if self.flat_buffer_size > offset else []
            slices = self.flat_param.split(self.param_sizes + pad)
            grad_slices = self.flat_grad.split(self.param_sizes + pad)
            with torch.no_grad():
                for p, dst, gdst in zip(self.param_list, slices, grad_slices):
                    dst = dst.view(p.shape)
                    dst.copy_(p.data)
                    p.data = dst
                    p.grad = gdst.view(p.shape)

        def state():
            return torch.zeros(self.shard_size, dtype=torch.float32, device=device)

        if skip_optimizer_step:
            self.flat_exp_avg_shard = self.flat_exp_avg_sq_shard = self.flat_fp32_master_param_shard = None
        else:
            self.flat_exp_avg_shard, self.flat_exp_avg_sq_shard = state(), state()
            self.flat_fp32_master_param_shard = self.flat_param_shard if dtype == torch.float32 \
                else self.flat_param_shard.to(torch.float32)
        self._norm_plan = GradNormPlan([0], [self.shard_size], device) if self.shard_size else None
        self._clip = torch.zeros(2, dtype=torch.float32, device=device)    # grad norm, clip multiplier

    def zero_grad(self):
        self.flat_grad.zero_()

    def _all_reduce_flat(self, tensor):
        parts = tensor.split(_ALLREDUCE_PART) if self.opt_use_chunked_allreduce else (tensor,)
        for part in parts:
            self.exchange.all_reduce(part, self.dp_group)

    def _accumulate_gradients(self, distributed):
        """Sum over the data-parallel ranks and average (optimizers.py:361-375)."""
        if not distributed or self.data_parallelism == 1:
            return
        if self.opt_use_allreduce_for_grad_acc:
            self._all_reduce_flat(self.flat_grad)
            self.flat_grad.div_(self.data_parallelism)
        else:
            self.exchange.reduce_scatter(self.flat_grad_shard, self.flat_grad, self.dp_group)
            self.flat_grad_shard.div_(self.data_parallelism)

    def shard_grad_norm(self):
        """Norm of this rank's gradient shard, rounded to the gradient dtype like
        torch.nn.utils.get_total_norm(flat_grad_shard) (optimizers.py:398); a 0-dim float32 device
        tensor that the next call overwrites."""
        return self._norm_plan.run(self.flat_grad_shard)[0]

    def _norm_and_multiplier(self, distributed):
        """optimizers.py:398-405 and :430-431: returns (grad_norm, multiplier) as device scalars."""
        shard_norm = self.shard_grad_norm()
        if distributed:
            value = shard_norm * shard_norm              # torch.pow(norm.float(), 2)
            self.exchange.all_reduce(value)              # over every rank of the job, like :402
        else:
            value = shard_norm
        _n.check(_n.lib().om_shard_clip_multiplier(
            _n.ptr(value), 1 if distributed else 0, _n.dtype_code(self.flat_grad), 1.0,
            _n.ptr(self._clip), _n.ptr(self._clip) + 4, _n.stream()), "om_shard_clip_multiplier")
        return self._clip[0], self._clip[1:2]

    def _gather_parameters(self, distributed):
        """Every rank ends the step with all updated parameters (optimizers.py:481-494)."""
        exchange = distributed and self.data_parallelism > 1
        if not self.opt_use_allreduce_for_param_gather:
            if exchange:
                self.exchange.all_gather(self.flat_param, self.flat_param_shard, self.dp_group)
            return
        lo = self.dp_ind * self.shard_size
        self.flat_param[:lo].zero_()
        self.flat_param[lo + self.shard_size:].zero_()
        if exchange:
            self._all_reduce_flat(self.flat_param)

    def step(self, closure=None):
        if self.dump_weight_gradients:
            raise NotImplementedError("dump_weight_gradients is a debugging aid outside this path")
        distributed = self.exchange.active()
        with record_pcl_function("4opt-step_1gradacc"):
            self._accumulate_gradients(distributed)
        if self.shard_size == 0:
            self.step_id += 1
            return torch.zeros((), dtype=torch.float32 if distributed else self.dtype, device=self.device)
        with record_pcl_function("4opt-step_3global-gradnorm"):
            grad_norm, multiplier = self._norm_and_multiplier(distributed)
        clip_now = self.opt_disable_delayed_grad_clipping or (self.step_id >= self.warmup_steps)
        with record_pcl_function("4opt-step_5compute"):
            if not (self.skip_optimizer_step or self.skip_optimizer_step_weight_update):
                group = self.param_groups[0]
                beta1, beta2 = self.defaults["betas"]
                adamw_step_(self.flat_param_shard, self.flat_grad_shard, self.flat_fp32_master_param_shard,
                            self.flat_exp_avg_shard, self.flat_exp_avg_sq_shard, self.step_id + 1,
                            group["lr"], beta1, beta2, self.defaults["eps"], self.defaults["weight_decay"],
                            grad_scale=multiplier if clip_now else None, store_scaled_grad=True)
            elif clip_now:
                scale_grad_(self.flat_grad_shard, multiplier)
        self._gather_parameters(distributed)
        self.step_id += 1
        # a fresh tensor: float32 after the all-reduce, the gradient dtype without a process group
        return grad_norm.to(torch.float32 if distributed else self.dtype, copy=True)

    def state_dict(self):
        state = {"step_id": self.step_id}
        if not self.disable_optimizer_state_checkpointing:
            for key in _SHARD_STATE_KEYS:
                state[key] = getattr(self, key)
        return state

    def load_state_dict(self, opt_state_dict):
        for key in _SHARD_STATE_KEYS:
            if key in opt_state_dict:
                getattr(self, key).copy_(opt_state_dict[key])
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


def scale_grad_(grad, coef):
    """grad = cast(grad * coef) in place, coef a device fp32 scalar: the multiply of
    clip_grads_with_norm_ (reference optimizers.py:145/150/154) for a tensor no update kernel reads."""
    _n.require_cuda_contiguous(grad, coef)
    if coef.dtype != torch.float32 or coef.numel() != 1:
        raise TypeError("coef must be one float32 element on the device")
    _n.check(_n.lib().om_grad_scale(_n.ptr(grad), grad.numel(), _n.dtype_code(grad), _n.ptr(coef),
                                    _n.stream()), "om_grad_scale")


def run_grad_norm(plan, flat_grad, foreign, cache, max_norm=1.0):
    """Total gradient norm and clip coefficient over flat_grad's parameters (through `plan`, may be
    None) followed by the tensors in `foreign`, each counted as one more parameter.  `cache` keeps
    the foreign tensors' chunk tables between steps."""
    if not foreign:
        return plan.run(flat_grad, max_norm)
    dtype = flat_grad.dtype
    for g in foreign:
        if g.dtype != dtype:
            raise TypeError("all gradients must share the optimizer's dtype")
    key = tuple((g.data_ptr(), g.numel()) for g in foreign)
    joint = cache.get(key)
    if joint is None:
        cache.clear()
        joint = cache[key] = JointGradNormPlan(plan, [g.numel() for g in foreign], flat_grad.device)
    return joint.run(flat_grad, foreign, max_norm)


class JointGradNormPlan:
    """One partial-sum table over flat_grad's chunks followed by the chunks of some separate
    gradient tensors; a single om_grad_norm_clip_coef over all of them."""

    def __init__(self, plan, foreign_sizes, device):
        self.flat = plan
        base_chunks = plan.n_chunks if plan is not None else 0
        first = plan.seg_first_chunk.cpu().tolist() if plan is not None else [0]
        self.tensors = []
        for size in foreign_sizes:
            sub = GradNormPlan([0], [size], device)
            self.tensors.append((sub, first[-1]))
            first.append(first[-1] + sub.n_chunks)
        self.n_chunks, self.n_segs = first[-1], len(first) - 1
        assert self.n_chunks >= base_chunks
        self.seg_first_chunk = torch.tensor(first, dtype=torch.int64).to(device)
        self.partials = torch.empty(max(self.n_chunks, 1), dtype=torch.float32, device=device)
        self.seg_norms = torch.empty(self.n_segs, dtype=torch.float32, device=device)
        self.out = torch.empty(2, dtype=torch.float32, device=device)

    def run(self, flat_grad, foreign, max_norm=1.0):
        lib = _n.lib()
        code = _n.dtype_code(flat_grad)
        if self.flat is not None:
            _n.check(lib.om_grad_sumsq(_n.ptr(flat_grad), code, _n.ptr(self.flat.chunk_offsets),
                                       self.flat.n_chunks, _n.ptr(self.partials), _n.stream()), "om_grad_sumsq")
        for g, (sub, at) in zip(foreign, self.tensors):
            _n.require_cuda_contiguous(g)
            _n.check(lib.om_grad_sumsq(_n.ptr(g), code, _n.ptr(sub.chunk_offsets), sub.n_chunks,
                                       _n.ptr(self.partials) + 4 * at, _n.stream()), "om_grad_sumsq")
        _n.check(lib.om_grad_norm_clip_coef(_n.ptr(self.partials), _n.ptr(self.seg_first_chunk),
                                            self.n_segs, code, float(max_norm), _n.ptr(self.seg_norms),
                                            _n.ptr(self.out), _n.ptr(self.out) + 4, _n.stream()),
                 "om_grad_norm_clip_coef")
        return self.out[0], self.out[1:2]
