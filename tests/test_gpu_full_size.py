"""The MoE layer at the full benchmark size (C3: 16384 tokens, hidden 2048, 64 experts, top-8, ffn
1024), checked through properties that hold exactly whatever the size, so no CPU reference of that
size is needed:
 * token permutation: routing, the expert MLP of a row and the weighted combine of a token do not
   depend on where the token sits, so permuting the input rows permutes output and input gradient.
   Not bit for bit: a tile starts its contraction at an offset that depends on the tile, so a row's
   fp32 sums are taken in another order when it lands in another tile, and now and then one of the
   bf16 roundings on the way falls the other side (measured: 0.5 % of the outputs and 1.7 % of the
   input gradients move, by one bf16 step); the same input twice gives the same bits;
 * scaling by a power of two is exact in bf16 and fp32, so doubling the down-projection weights
   doubles the output exactly, and doubling the output gradient doubles every gradient exactly;
 * index construction: the permutation arrays invert each other, rows are grouped by ascending
   expert and, inside an expert, by ascending token; counts add up to T*K."""
import pytest
import torch

import synthetic_configs as sc

pytestmark = pytest.mark.gpu


def _block(inp, cuda):
    from test_gpu_moe_layer import _olmoe_block
    return _olmoe_block(inp, cuda)


def _run(blk, x, dout):
    for p in blk.parameters():
        p.grad = None
    xg = x.clone().requires_grad_(True)
    out, _ = blk(xg.view(4, -1, x.shape[-1]))
    out.backward(dout.view_as(out))
    grads = {n: p.grad.clone() for n, p in blk.named_parameters()}
    return out.detach().reshape(x.shape), xg.grad.clone(), grads


def test_c3_full_size_permutation_and_scaling(cuda):
    inp = sc.moe_inputs("C3")
    T = inp["cfg"]["T"]
    blk = _block(inp, cuda)
    x = inp["x"].to(cuda); dout = inp["dout"].to(cuda)
    out, dx, grads = _run(blk, x, dout)
    assert torch.isfinite(out.float()).all() and float(out.float().abs().mean()) > 0

    perm = torch.randperm(T, generator=torch.Generator().manual_seed(5)).to(cuda)
    out_p, dx_p, grads_p = _run(blk, x[perm], dout[perm])
    for got, want in ((out_p, out[perm]), (dx_p, dx[perm])):
        d = (got.float() - want.float()).abs()
        assert float((d > 0).float().mean()) <= 0.03
        assert float(d.max()) <= 2.0 ** -7 * float(want.float().abs().max())
    out_r, dx_r, grads_r = _run(blk, x, dout)          # run-to-run: identical bits
    assert torch.equal(out_r, out) and torch.equal(dx_r, dx)
    assert all(torch.equal(grads_r[n], grads[n]) for n in grads)
    # weight gradients sum the same terms in another order: equal up to bf16 rounding of the sums
    for n in grads:
        a, b = grads_p[n].float(), grads[n].float()
        assert float((a - b).abs().max()) <= 2e-2 * float(b.abs().max()), n

    out_2, dx_2, grads_2 = _run(blk, x, dout * 2)
    assert torch.equal(out_2, out) and torch.equal(dx_2, dx * 2)
    for n in grads:
        assert torch.equal(grads_2[n], grads[n] * 2), n

    with torch.no_grad():
        blk.experts.down_proj_merged_weight.mul_(2)
    out_w, _, _ = _run(blk, x, dout)
    assert torch.equal(out_w, out * 2)


def test_c3_full_size_index_construction(cuda):
    from optimus.models.common.moe import SoftmaxTopkRouterFunction, build_token_permutation
    inp = sc.moe_inputs("C3")
    c = inp["cfg"]
    T, K, N = c["T"], c["K"], c["N"]
    logits = (inp["x"].float() @ inp["gate_w"].float().t()).to(cuda)
    _, experts = SoftmaxTopkRouterFunction.apply(logits, K, False, torch.bfloat16)
    cum, cum_ep, input_indices, output_indices, sel_idx = build_token_permutation(experts, 0, N)
    cum = cum.cpu().long(); TR = int(cum[-1])
    assert TR == T * K and bool((cum[1:] >= cum[:-1]).all())
    assert torch.equal(cum[1:] - cum[:-1], torch.bincount(experts.flatten().cpu(), minlength=N))
    ii = input_indices[:TR].long(); oi = output_indices[:TR].long()
    # output_indices is a permutation of the rows, and the row of pair j belongs to token j // K
    assert torch.equal(torch.sort(oi).values, torch.arange(TR, device=cuda))
    assert torch.equal(ii[oi], torch.arange(TR, device=cuda) // K)
    assert torch.equal(sel_idx[:TR].long(), torch.arange(TR, device=cuda) % K)
    # rows are grouped by expert (ascending) and ordered by token inside an expert
    row_expert = torch.bucketize(torch.arange(TR), cum[1:], right=True).to(cuda)
    assert torch.equal(experts.flatten()[torch.argsort(oi)], row_expert)
    same = row_expert[1:] == row_expert[:-1]
    assert bool((ii[1:][same] > ii[:-1][same]).all())
    assert torch.equal(cum_ep.cpu().long(), torch.arange(T + 1) * K)


def test_c5_full_size_one_rank_share(cuda):
    """C5 at its real shape: 8192 tokens, hidden 7168, this rank's 32 of 256 routed experts (ffn 2048)
    plus the shared expert.  Same properties: determinism, permutation, exact scaling."""
    from optimus.mapper import ParallelDpPpEpTpMapper
    from optimus.models.deepseek_v3.configuration_deepseek_v3 import DeepseekV3ParallelConfig
    from optimus.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3ParallelMoE
    inp = sc.dsv3_inputs()
    c = inp["cfg"]
    T, H = c["T"], c["H"]
    cfg = DeepseekV3ParallelConfig(expert_parallelism=8)
    assert (cfg.hidden_size, cfg.moe_intermediate_size, cfg.n_routed_experts) == (H, c["I"], c["N"])
    blk = DeepseekV3ParallelMoE(cfg, ParallelDpPpEpTpMapper(expert_parallelism=8, rank=2)).to(cuda).to(torch.bfloat16)
    with torch.no_grad():
        blk.gate.weight.copy_(inp["router_w"]); blk.gate.e_score_correction_bias.copy_(inp["bias"])
        for e, m in enumerate(blk.experts):
            m.gate_proj.weight.copy_(inp["w_gate"][e]); m.up_proj.weight.copy_(inp["w_up"][e])
            m.down_proj.weight.copy_(inp["w_down"][e])
        blk.shared_experts.gate_proj.weight.copy_(inp["ws_gate"]); blk.shared_experts.up_proj.weight.copy_(inp["ws_up"])
        blk.shared_experts.down_proj.weight.copy_(inp["ws_down"])
    x = inp["x"].to(cuda); dout = inp["dout"].to(cuda)

    def run(xx, dd):
        for p in blk.parameters():
            p.grad = None
        xg = xx.clone().requires_grad_(True)
        out = blk(xg.view(2, T // 2, H))
        out.backward(dd.view_as(out))
        return out.detach().reshape(T, H), xg.grad.clone()

    out, dx = run(x, dout)
    e, w = blk.gate(x)
    local = ((e >= 64) & (e < 96)).sum()
    assert torch.isfinite(out.float()).all() and int(local) > 0.8 * T      # about T routed rows on this rank
    out_r, dx_r = run(x, dout)
    assert torch.equal(out_r, out) and torch.equal(dx_r, dx)
    perm = torch.randperm(T, generator=torch.Generator().manual_seed(6)).to(cuda)
    out_p, dx_p = run(x[perm], dout[perm])
    for got, want in ((out_p, out[perm]), (dx_p, dx[perm])):
        d = (got.float() - want.float()).abs()
        assert float((d > 0).float().mean()) <= 0.05
        assert float(d.max()) <= 2.0 ** -6 * float(want.float().abs().max())
    out_2, dx_2 = run(x, dout * 2)
    assert torch.equal(out_2, out) and torch.equal(dx_2, dx * 2)
