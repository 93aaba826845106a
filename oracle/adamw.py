"""AdamW restatements.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

adamw_step_torch   — the reference's chunked sequence of torch elementwise ops,
                     optimus/optimizers.py:162-205, on CPU tensors.  This is the "port" that
                     bench.py times as cpu_baseline for the AdamW workload.
sharded_clip_and_step_torch — ShardedMixedPrecisionAdamW.step from the accumulated gradient shards
                     on (optimus/optimizers.py:398-479) for all ranks at once, collectives replaced
                     by their definitions.
The scalar C versions (fp32 op-by-op and fp64) are in oracle/adamw_oracle.c via oracle/clib.py.
"""
import math

import torch


def adamw_step_torch(flat_param, flat_grad, flat_master, flat_exp_avg, flat_exp_avg_sq, step_id,
                     lr, betas, eps, weight_decay, chunk_size=128 * 1024 * 1024):
    """In place; step_id is 0-based like MixedPrecisionAdamW.step_id (t = step_id + 1)."""
    beta1, beta2 = betas
    size = flat_param.numel()
    num_chunks = math.ceil(size / chunk_size)                                    # :179-180
    tensor_list = [flat_param, flat_grad, flat_master, flat_exp_avg, flat_exp_avg_sq]
    for chunk_id in range(num_chunks):
        s = chunk_id * chunk_size
        e = min((chunk_id + 1) * chunk_size, size)
        data, grad, master, exp_avg, exp_avg_sq = [t[s:e] for t in tensor_list]
        g32 = grad.to(torch.float32)                                             # :190
        exp_avg.mul_(beta1).add_(g32, alpha=(1.0 - beta1))                       # :193
        exp_avg_sq.mul_(beta2).addcmul_(g32, g32, value=1.0 - beta2)             # :194
        exp_avg_hat = exp_avg / (1.0 - math.pow(beta1, (step_id + 1)))           # :195
        exp_avg_sq_hat = exp_avg_sq / (1.0 - math.pow(beta2, (step_id + 1)))     # :196
        denom = exp_avg_sq_hat.sqrt().add_(eps)                                  # :197
        master.addcdiv_(exp_avg_hat, denom, value=-lr)                           # :198
        if weight_decay > 0.0:
            master.add_(master, alpha=(-lr * weight_decay))                      # :202
        data.copy_(master.to(data.dtype))                                        # :205


def grad_norm_and_clip_torch(grads, clip, max_norm=1.0):
    """The reference's gradient-norm block for one device, optimus/optimizers.py:136-160: the
    norm is always taken (`get_total_norm`), the clip (`clip_grads_with_norm_`, equivalently
    `clip_grad_norm_`) only when `clip`.  `grads` are CPU tensors, scaled in place.  These are
    the library calls the reference makes, so this is the pin for the scalar C restatement."""
    total = torch.nn.utils.get_total_norm(grads)                                  # :147/:156
    if clip:
        holders = [torch.nn.Parameter(torch.empty_like(g)) for g in grads]
        for h, g in zip(holders, grads):
            h.grad = g
        torch.nn.utils.clip_grads_with_norm_(holders, max_norm, total)           # :148
    return total


def sharded_clip_and_step_torch(grad_shards, param_shards, master_shards, exp_avg_shards, exp_avg_sq_shards,
                                step_id, lr, betas, eps, weight_decay, clip, process_group, max_norm=1.0):
    """ShardedMixedPrecisionAdamW.step (optimus/optimizers.py:398-479) for every rank of a job at
    once, on CPU tensors, in place; rank r owns element r of each list.  The gradient shards are
    taken as already accumulated (the reduce-scatter's summation order belongs to the collective).
    `process_group` False is the single-process branch (:404-405; one rank only).
    Two things are made explicit that the device run of the reference does implicitly:
      * all_reduce(sum) of the squared norms = the ranks' values added in rank order;
      * `flat_grad_shard.mul_(clip_coef)` with both operands on the device casts the 0-dim float32
        coefficient to the gradient dtype before multiplying (on CPU tensors torch would take a 0-dim
        operand as an exact scalar), hence `.to(g.dtype)` below.
    Returns grad_norm as the reference's step does."""
    norms = [torch.nn.utils.get_total_norm(g) for g in grad_shards]               # :398
    if process_group:
        total = None
        for n in norms:
            sq = torch.pow(n.to(torch.float32), 2)                                # :400-401
            total = sq if total is None else total + sq                           # :402
        grad_norm = torch.sqrt(total)                                             # :403
    else:
        assert len(grad_shards) == 1
        grad_norm = norms[0]                                                      # :405
    if clip:
        clip_coef = max_norm / (grad_norm + 1e-6)                                 # :430
        if clip_coef < 1.0:                                                       # :431
            for g in grad_shards:
                g.mul_(clip_coef.to(g.dtype))                                     # :432
    for r in range(len(grad_shards)):                                             # :434-479
        adamw_step_torch(param_shards[r], grad_shards[r], master_shards[r], exp_avg_shards[r],
                         exp_avg_sq_shards[r], step_id, lr, betas, eps, weight_decay)
    return grad_norm
