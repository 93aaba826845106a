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


# ----------------------------------------------------------------------------------------------
# The full-size layers against the fp32 oracle on a SAMPLE: the layer is a per-token function
# (out[t] = sum_k w[t,k] MLP_e[t,k](x[t]) (+ shared MLP), reference modeling_olmoe.py:322-336,
# modeling_deepseek_v3.py:221-265), so the oracle evaluated on a few hundred tokens gives those
# tokens' rows of the full-size output and input gradient exactly; an expert's weight gradient
# needs only the tokens routed to it, so two or three experts are affordable on the CPU.
# ----------------------------------------------------------------------------------------------
from oracle import moe_layer as L      # noqa: E402
from oracle import routing as R        # noqa: E402
from util import assert_bf16_parity    # noqa: E402

# measured: out 1.95-2.29 x the bf16 floor, dx 2.8-3.2 x, d routing weights 2.5 x, expert dW 1.4-2.7 x
SAMPLE_BARS = {"out": (2.6, 3.5e-3), "grad": (3.5, 5e-3), "wgrad": (3.2, 4.5e-3)}


def _expert_wgrads(x, dout, tok, w_tok, wg, wu, wd):
    """dW_gate, dW_up, dW_down of ONE expert from first principles: autograd through
    w * MLP(x[tok]) for the tokens routed to it (all of them: nothing else touches its weights)."""
    p = [t.float().requires_grad_(True) for t in (wg, wu, wd)]
    if tok.numel():
        y = L.expert_mlp(x[tok].float(), *p) * w_tok[:, None]
        y.backward(dout[tok].float())
    return [t.grad if t.grad is not None else torch.zeros_like(t) for t in p]


def test_c3_full_size_sampled_against_oracle(cuda, monkeypatch):
    """C3 at 16384 x 2048, 64 experts, top-8: router ids of all tokens bit-exact; output rows, input
    gradient rows and routing-weight gradients of 256 sampled tokens, and the three weight gradients
    of the most and the least loaded expert, against the fp32 oracle."""
    from optimus.models.common import moe as M
    inp = sc.moe_inputs("C3")
    c = inp["cfg"]
    T, H, K, N = c["T"], c["H"], c["K"], c["N"]
    blk = _block(inp, cuda)
    seen = {}
    real = M.expert_computation

    def spy(hidden_states, routing_weights, selected_experts, *a, **kw):
        routing_weights.retain_grad()
        seen["w"], seen["e"] = routing_weights, selected_experts
        return real(hidden_states, routing_weights, selected_experts, *a, **kw)

    monkeypatch.setattr(M, "expert_computation", spy)
    xg = inp["x"].to(cuda).requires_grad_(True)
    out, _ = blk(xg.view(4, -1, H))
    out.backward(inp["dout"].to(cuda).view_as(out))
    torch.cuda.synchronize()
    out = out.detach().reshape(T, H).cpu(); dx = xg.grad.cpu()
    e_gpu = seen["e"].cpu(); dw_gpu = seen["w"].grad.float().cpu()

    # router on the CPU for every token
    logits = inp["x"].float() @ inp["gate_w"].float().t()
    _, e_ref, probs = R.olmoe_router(logits, K, False, torch.float32)
    top = torch.sort(probs, dim=1, descending=True).values[:, :K + 1]
    gap_ulps = ((top[:, :-1] - top[:, 1:]) / (top[:, :-1] * 2.0 ** -23)).min(1).values
    assert float(gap_ulps.min()) > 4.0, "fixture invalid: reseed"
    safe = gap_ulps > 64.0               # rows that no summation order of the 2048-term logits can reorder
    assert float(safe.float().mean()) > 0.999
    assert torch.equal(e_gpu[safe], e_ref[safe])
    # the few rows outside `safe` may order or cut a near-tie differently: at most one expert differs
    differ = (torch.sort(e_gpu[~safe], 1).values != torch.sort(e_ref[~safe], 1).values).any(1)
    for a, b in zip(e_gpu[~safe][differ].tolist(), e_ref[~safe][differ].tolist()):
        assert len(set(a) & set(b)) >= K - 1
    w_use = probs.gather(1, e_gpu)       # the rows outside `safe` take the GPU's (equally valid) order

    # 256 sampled tokens: the whole layer in fp32 with autograd
    idx = torch.nonzero(safe).flatten()
    idx = idx[torch.randperm(idx.numel(), generator=torch.Generator().manual_seed(11))[:256]].sort().values
    wf = {k: inp[k].float() for k in ("gate_w", "w_gate", "w_up", "w_down")}
    xs = inp["x"][idx].float().requires_grad_(True)
    lg = torch.nn.functional.linear(xs, wf["gate_w"])
    w_s, e_s, _ = R.olmoe_router(lg, K, False, torch.float32)
    w_s.retain_grad()
    assert torch.equal(e_s, e_gpu[idx])
    ref = torch.zeros(idx.numel(), H)
    for n in range(N):
        tok, kk = torch.where(e_s == n)
        if tok.numel():
            y = L.expert_mlp(xs[tok], wf["w_gate"][n], wf["w_up"][n], wf["w_down"][n])
            ref = ref.index_add(0, tok, y * w_s[tok, kk, None])
    ref.backward(inp["dout"][idx].float())
    assert_bf16_parity(out[idx], ref, *SAMPLE_BARS["out"], tag="C3 full sampled out", max_abs_bar=2e-2)
    assert_bf16_parity(dx[idx], xs.grad, *SAMPLE_BARS["grad"], tag="C3 full sampled dx")
    assert_bf16_parity(dw_gpu[idx], w_s.grad, *SAMPLE_BARS["grad"], tag="C3 full sampled d routing_weights")

    # weight gradients of the heaviest and the lightest expert, over all their tokens
    counts = torch.bincount(e_gpu.flatten(), minlength=N)
    grads = {"w_gate": blk.experts.gate_proj_merged_weight.grad, "w_up": blk.experts.up_proj_merged_weight.grad,
             "w_down": blk.experts.down_proj_merged_weight.grad}
    for n in (int(counts.argmax()), int(counts.argmin())):
        tok, kk = torch.where(e_gpu == n)
        want = _expert_wgrads(inp["x"], inp["dout"], tok, w_use[tok, kk], inp["w_gate"][n], inp["w_up"][n],
                              inp["w_down"][n])
        for (name, g), wnt in zip(grads.items(), want):
            assert_bf16_parity(g[n], wnt, *SAMPLE_BARS["wgrad"], tag=f"C3 full expert {n} ({int(counts[n])} rows) d{name}")


class _FloatOnDemand:
    """Stacked per-expert bf16 weights that hand out one expert at a time as float32 (the oracle
    indexes `w[i]` and reads `w.shape[0]`); avoids a float32 copy of all 32 x 88 MB matrices."""

    def __init__(self, t):
        self.t, self.shape = t, t.shape

    def __getitem__(self, i):
        return self.t[i].float()


def test_c5_full_size_sampled_against_oracle(cuda):
    """C5 at its real shape (8192 x 7168, 32 local of 256 experts, ffn 2048, shared expert): expert
    sets of all tokens with a safe selection margin identical to the oracle's; output rows and
    input-gradient rows of 192 sampled tokens against oracle.moe_layer.dsv3_moe_block; weight
    gradients of the heaviest, a light and an empty local expert from first principles."""
    from optimus.mapper import ParallelDpPpEpTpMapper
    from optimus.models.deepseek_v3.configuration_deepseek_v3 import DeepseekV3ParallelConfig
    from optimus.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3ParallelMoE
    inp = sc.dsv3_inputs()
    c = inp["cfg"]
    T, H, K, NR, rank = c["T"], c["H"], c["K"], c["NR"], 2
    start = rank * NR
    cfg = DeepseekV3ParallelConfig(expert_parallelism=8)
    blk = DeepseekV3ParallelMoE(cfg, ParallelDpPpEpTpMapper(expert_parallelism=8, rank=rank)).to(cuda).to(torch.bfloat16)
    with torch.no_grad():
        blk.gate.weight.copy_(inp["router_w"]); blk.gate.e_score_correction_bias.copy_(inp["bias"])
        for e, m in enumerate(blk.experts):
            m.gate_proj.weight.copy_(inp["w_gate"][e]); m.up_proj.weight.copy_(inp["w_up"][e])
            m.down_proj.weight.copy_(inp["w_down"][e])
        blk.shared_experts.gate_proj.weight.copy_(inp["ws_gate"]); blk.shared_experts.up_proj.weight.copy_(inp["ws_up"])
        blk.shared_experts.down_proj.weight.copy_(inp["ws_down"])
    xg = inp["x"].to(cuda).requires_grad_(True)
    out = blk(xg.view(2, T // 2, H))
    out.backward(inp["dout"].to(cuda).view_as(out))
    e_gpu, _ = blk.gate(xg.detach())
    torch.cuda.synchronize()
    out = out.detach().reshape(T, H).cpu(); dx = xg.grad.cpu(); e_gpu = e_gpu.cpu()

    rw = inp["router_w"].to(torch.bfloat16).float()          # the module holds the router weight in bf16
    bias = blk.gate.e_score_correction_bias.detach().float().cpu()
    scores64 = torch.sigmoid(inp["x"].double() @ rw.double().t())
    margin = R.dsv3_selection_margin(scores64, bias.double(), c["n_group"], c["topk_group"], K)
    safe = margin > 2e-6
    assert float(safe.float().mean()) > 0.995
    e_ref, _ = R.dsv3_topk_indices(scores64, bias.double(), c["n_group"], c["topk_group"], K)
    assert torch.equal(torch.sort(e_gpu, 1).values[safe], torch.sort(e_ref, 1).values[safe])

    idx = torch.nonzero(safe).flatten()
    idx = idx[torch.randperm(idx.numel(), generator=torch.Generator().manual_seed(12))[:192]].sort().values
    xs = inp["x"][idx].float().requires_grad_(True)
    ref, e_s, w_s = L.dsv3_moe_block(xs, rw, bias, _FloatOnDemand(inp["w_gate"]), _FloatOnDemand(inp["w_up"]),
                                     _FloatOnDemand(inp["w_down"]), inp["ws_gate"].float(), inp["ws_up"].float(),
                                     inp["ws_down"].float(), c["n_group"], c["topk_group"], K, True, 2.5,
                                     expert_start_idx=start)
    assert torch.equal(torch.sort(e_s, 1).values, torch.sort(e_gpu[idx], 1).values)
    assert int(((e_s >= start) & (e_s < start + NR)).sum()) > 100     # the sample does exercise the routed experts
    ref.backward(inp["dout"][idx].float())
    assert_bf16_parity(out[idx], ref, *SAMPLE_BARS["out"], tag="C5 full sampled out", max_abs_bar=2e-2)
    assert_bf16_parity(dx[idx], xs.grad, *SAMPLE_BARS["grad"], tag="C5 full sampled dx")

    # weights of the GPU's own (valid) selection, from the fp32 scores as the reference forms them
    scores = scores64.float()
    w_all = scores.gather(1, e_gpu)
    w_all = w_all / (w_all.sum(1, keepdim=True) + 1e-20) * 2.5
    local = e_gpu - start
    counts = torch.bincount(local[(local >= 0) & (local < NR)].flatten(), minlength=NR)
    heavy = int(counts.argmax())
    light = int(torch.where(counts > 0, counts, torch.full_like(counts, 1 << 30)).argmin())
    picks = [heavy, light] + ([int(torch.nonzero(counts == 0)[0])] if bool((counts == 0).any()) else [])
    for n in picks:
        tok, kk = torch.where(local == n)
        want = _expert_wgrads(inp["x"], inp["dout"], tok, w_all[tok, kk], inp["w_gate"][n], inp["w_up"][n],
                              inp["w_down"][n])
        m = blk.experts[n]
        for name, g, wnt in zip(("w_gate", "w_up", "w_down"),
                                (m.gate_proj.weight.grad, m.up_proj.weight.grad, m.down_proj.weight.grad), want):
            if int(counts[n]) == 0:
                assert float(g.float().abs().max()) == 0.0
            else:
                assert_bf16_parity(g, wnt, *SAMPLE_BARS["wgrad"], tag=f"C5 full expert {n} ({int(counts[n])} rows) d{name}")
