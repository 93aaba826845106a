"""The bf16 tolerance anchored to the reference's own numerics.

oracle.moe_layer.fast_block_sequence evaluates the reference's operator sequence for the expert half of
the fast block (K4 gather -> MergedMLP.forward -> K6 combine, optimus/models/common/moe.py:217-405,
gradients through exactly those operators) once in float32 and once in bfloat16 with every rounding
that sequence has.  The distance of the bfloat16 evaluation from the float32 one is what the
reference's own path loses; the HIP path must not lose more than that, for the output and
for every gradient.  The routing (weights and experts) is computed once on the CPU and given to both
sides, so only the expert path is compared.
"""
import pytest
import torch

import synthetic_configs as sc
from oracle import moe_layer as L
from oracle import routing as R
from util import mean_rel

pytestmark = pytest.mark.gpu

ALLOWED = 1.0     # times the reference sequence's own distance from float32 (measured: 0.54-0.92)
_cpu_side = {}    # config name -> the two CPU evaluations (shared by the two GPU forms)


def _gpu_expert_path(cuda, inp, w, e, fuse):
    from optimus.models.common.moe import MergedMLPFunction, RoutedMLPFunction, expert_computation
    c = inp["cfg"]
    t = {k: inp[k].to(cuda).requires_grad_(True) for k in ("x", "w_gate", "w_up", "w_down")}
    wd = w.to(cuda).requires_grad_(True)
    fn = lambda gi, cum: MergedMLPFunction.apply(gi, t["w_gate"], t["w_up"], t["w_down"], cum)
    routed = None
    if fuse:
        routed = lambda hs, rw, ii, cum_ep, oi, si, cum, res: RoutedMLPFunction.apply(
            hs, rw, ii, cum_ep, oi, si, cum, res, True, t["w_gate"], t["w_up"], t["w_down"])
    out = expert_computation(t["x"], wd, e.to(cuda), 0, c["N"], fn, c["N"], routed_experts_fn=routed)
    out.backward(inp["dout"].to(cuda))
    torch.cuda.synchronize()
    grads = {k: v.grad.float().cpu() for k, v in t.items()}
    grads["routing_weights"] = wd.grad.float().cpu()
    return out.detach().float().cpu(), grads


@pytest.mark.parametrize("name,scale", [("C1", 1.0), ("C3", 0.125), ("C4", 1.0)])
@pytest.mark.parametrize("fuse", [False, True], ids=["separate_functions", "routing_weight_in_mlp"])
def test_not_further_from_float32_than_the_reference_sequence_in_bf16(cuda, name, scale, fuse):
    inp = sc.moe_inputs(name, scale_tokens=scale)
    c = inp["cfg"]
    logits = inp["logits"] if inp["logits"] is not None else inp["x"].float() @ inp["gate_w"].float().t()
    w, e, _ = R.olmoe_router(logits, c["K"], c["norm_topk_prob"], torch.bfloat16)
    args = ("x", "w_gate", "w_up", "w_down")
    if name not in _cpu_side:
        f32 = lambda k: inp[k].float()
        _cpu_side[name] = (
            L.fast_block_sequence(f32("x"), w.float(), e, f32("w_gate"), f32("w_up"), f32("w_down"),
                                  inp["dout"].float()),
            L.fast_block_sequence(inp["x"], w, e, inp["w_gate"], inp["w_up"], inp["w_down"], inp["dout"]))
    (ref_out, ref), (seq_out, seq) = _cpu_side[name]
    gpu_out, gpu = _gpu_expert_path(cuda, inp, w, e, fuse)
    rows = [("out", gpu_out, seq_out.float(), ref_out)]
    rows += [("d" + k, gpu[k], seq[k].float(), ref[k]) for k in args + ("routing_weights",)]
    report = []
    for tag, got, reference_bf16, exact in rows:
        ours, theirs = mean_rel(got, exact), mean_rel(reference_bf16, exact)
        report.append((tag, ours, theirs, ours / theirs))
    worst = max(report, key=lambda r: r[3])
    print("\n".join(f"{name} fuse={fuse} {t:18s} hip {a:.3e} reference-bf16 {b:.3e} ratio {r:.3f}" for t, a, b, r in report))
    assert worst[3] <= ALLOWED, report
