"""Whole-layer parity of the MoE modules against the fp32 restatement of the reference blocks.

Bar (north star): expert indices bit-exact; outputs and gradients max-abs <= 2e-2 and mean-rel
<= 1e-3 against the fp32 reference evaluated on the same bf16-rounded inputs (mean_rel :=
mean|a-b| / mean|b|)."""
import numpy as np
import pytest
import torch

import synthetic_configs as sc
from oracle import moe_layer as L
from oracle import routing as R
from util import max_abs, mean_rel

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 1e-3


def _olmoe_block(inp, cuda, fast=True, merged=True, fp32_logits=True):
    from optimus.mapper import ParallelDpPpEpTpMapper
    from optimus.models.common.moe import FastOlmoeParallelSparseMoeBlock
    from optimus.models.olmoe.configuration_olmoe import OlmoeParallelConfig
    from optimus.models.olmoe.modeling_olmoe import OlmoeParallelSparseMoeBlock
    c = inp["cfg"]
    cfg = OlmoeParallelConfig(hidden_size=c["H"], intermediate_size=c["I"], num_experts=c["N"],
                              num_experts_per_tok=c["K"], norm_topk_prob=c["norm_topk_prob"],
                              output_router_logits=True, use_fast_moe=fast,
                              use_merged_mlp_in_fast_moe=merged)
    cfg.router_logits_fp32 = fp32_logits
    cls = FastOlmoeParallelSparseMoeBlock if fast else OlmoeParallelSparseMoeBlock
    blk = cls(cfg, ParallelDpPpEpTpMapper()).to(cuda).to(torch.bfloat16)
    with torch.no_grad():
        blk.gate.weight.copy_(inp["gate_w"])
        if fast and merged:
            blk.experts.gate_proj_merged_weight.copy_(inp["w_gate"])
            blk.experts.up_proj_merged_weight.copy_(inp["w_up"])
            blk.experts.down_proj_merged_weight.copy_(inp["w_down"])
        else:
            for e, m in enumerate(blk.experts):
                m.gate_proj.weight.copy_(inp["w_gate"][e])
                m.up_proj.weight.copy_(inp["w_up"][e])
                m.down_proj.weight.copy_(inp["w_down"][e])
    return blk


def _reference(inp):
    """fp32 slow block + autograd on the bf16-rounded inputs."""
    c = inp["cfg"]
    t = {k: inp[k].float().requires_grad_(True) for k in ("x", "gate_w", "w_gate", "w_up", "w_down")}
    out, logits = L.olmoe_slow_block(t["x"], t["gate_w"], t["w_gate"], t["w_up"], t["w_down"], c["K"],
                                     c["norm_topk_prob"])
    out.backward(inp["dout"].float())
    return out.detach(), logits.detach(), {k: v.grad for k, v in t.items()}


@pytest.mark.parametrize("name,scale", [("C1", 1.0), ("C3", 0.125), ("C4", 1.0)])
def test_fast_block_fwd_bwd(cuda, name, scale):
    inp = sc.moe_inputs(name, scale_tokens=scale)
    if inp["logits"] is not None:
        pytest.skip("C4 injects router logits; covered by test_fast_block_injected_logits")
    c = inp["cfg"]
    ref_out, ref_logits, ref_grads = _reference(inp)
    assert R.min_topk_gap_ulps(torch.softmax(ref_logits, 1), c["K"]) > 4.0, "fixture invalid: reseed"
    blk = _olmoe_block(inp, cuda)
    x = inp["x"].to(cuda).view(1, c["T"], c["H"]).requires_grad_(True)
    out, logits = blk(x)
    out.backward(inp["dout"].to(cuda).view_as(out))
    torch.cuda.synchronize()
    # routing decisions identical
    _, e_ref, _ = R.olmoe_router(ref_logits, c["K"], c["norm_topk_prob"], torch.float32)
    _, e_gpu, _ = R.olmoe_router(logits.float().cpu(), c["K"], c["norm_topk_prob"], torch.float32)
    assert torch.equal(e_ref, e_gpu)
    o = out.float().cpu().view(c["T"], c["H"])
    assert max_abs(o, ref_out) <= MAX_ABS and mean_rel(o, ref_out) <= 4e-3, (max_abs(o, ref_out), mean_rel(o, ref_out))
    got = {"x": x.grad.view(c["T"], c["H"]), "gate_w": blk.gate.weight.grad,
           "w_gate": blk.experts.gate_proj_merged_weight.grad, "w_up": blk.experts.up_proj_merged_weight.grad,
           "w_down": blk.experts.down_proj_merged_weight.grad}
    for k, gref in ref_grads.items():
        a = got[k].float().cpu()
        assert mean_rel(a, gref) <= 1e-2, (k, mean_rel(a, gref))
        assert max_abs(a, gref) <= MAX_ABS * max(1.0, float(gref.abs().max())), (k, max_abs(a, gref))
