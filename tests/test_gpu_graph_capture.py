"""The MoE block's forward and backward recorded once into a HIP graph and replayed.

The library's entry points only enqueue kernels on the stream they are given (no allocation, no
synchronisation, no memset) and, without an expert window, the host side never reads a device
value, so a whole layer step can be captured.  Each replay is checked bit for bit against an eager
run of a second block with the same weights on the same inputs; the replays are separated by eager
work and synchronisations, and inputs change between them."""
import copy

import pytest
import torch

import synthetic_configs as sc

pytestmark = pytest.mark.gpu


def _block(inp, cuda):
    from test_gpu_moe_layer import _olmoe_block
    return _olmoe_block(inp, cuda)


def _grads(blk):
    return {n: p.grad.clone() for n, p in blk.named_parameters() if p.grad is not None}


@pytest.mark.parametrize("name,scale", [("C1", 1.0), ("C3", 1.0 / 32)])
def test_layer_step_replays_from_a_graph(cuda, name, scale):
    inp = sc.moe_inputs(name, scale_tokens=scale)
    c = inp["cfg"]
    graphed = _block(inp, cuda)
    eager = copy.deepcopy(graphed)
    shape = (1, c["T"], c["H"])
    x_static = inp["x"].to(cuda).view(shape).clone().requires_grad_(True)
    dout_static = inp["dout"].to(cuda).view(shape).clone()

    def step(blk, x, dout):
        out, logits = blk(x)
        out.backward(dout)
        return out, logits

    # torch's recipe: warm up on a side stream, then capture with the gradients unset so that the
    # backward allocates them from the graph's own pool
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(graphed, x_static, dout_static)
    torch.cuda.current_stream().wait_stream(side)
    graphed.zero_grad(set_to_none=True)
    x_static.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static, logits_static = step(graphed, x_static, dout_static)

    gen = torch.Generator().manual_seed(5)
    for trial in range(4):
        if trial:
            with torch.no_grad():
                x_static.copy_(torch.randn(shape, generator=gen).to(torch.bfloat16))
                dout_static.copy_(torch.randn(shape, generator=gen).to(torch.bfloat16))
        graph.replay()
        torch.cuda.synchronize()
        # eager run of the twin on the same inputs (also the "program's own work" between replays)
        eager.zero_grad(set_to_none=True)
        x = x_static.detach().clone().requires_grad_(True)
        out, logits = step(eager, x, dout_static)
        torch.cuda.synchronize()
        assert torch.equal(out_static, out), trial
        assert torch.equal(logits_static, logits), trial
        assert torch.equal(x_static.grad, x.grad), trial
        want = _grads(eager)
        got = _grads(graphed)
        assert set(got) == set(want) and len(got) >= 4
        for k in want:
            assert torch.equal(got[k], want[k]), (trial, k)


def _dsv3_window_block(cuda, sync_free, ep_ind=1, seed=7):
    from optimus.mapper import ParallelDpPpEpTpMapper
    from optimus.models.deepseek_v3.configuration_deepseek_v3 import DeepseekV3ParallelConfig
    from optimus.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3ParallelMoE
    cfg = DeepseekV3ParallelConfig(hidden_size=512, moe_intermediate_size=256, n_routed_experts=64,
                                   num_experts_per_tok=8, n_group=8, topk_group=4, expert_parallelism=4)
    cfg.sync_free_expert_window = sync_free
    torch.manual_seed(seed)
    blk = DeepseekV3ParallelMoE(cfg, ParallelDpPpEpTpMapper(expert_parallelism=4, rank=ep_ind))
    for p in blk.parameters():
        torch.nn.init.normal_(p, std=0.03)
    torch.nn.init.normal_(blk.gate.e_score_correction_bias, std=0.1)
    return blk.to(cuda).to(torch.bfloat16)


def test_window_without_host_read_gives_the_same_bits(cuda):
    """An expert window with the routed-row count left on the device (index arrays and expert
    activations sized by T*K) against the default that reads the count back like the reference
    (moe.py:520): outputs and every gradient bit-identical, including the zero routing-weight
    gradient of the pairs routed to other ranks."""
    a = _dsv3_window_block(cuda, False)
    b = _dsv3_window_block(cuda, True)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 300, 512, generator=g).to(torch.bfloat16).to(cuda)
    d = torch.randn(2, 300, 512, generator=g).to(torch.bfloat16).to(cuda)
    res = []
    for blk in (a, b):
        xi = x.clone().requires_grad_(True)
        out = blk(xi)
        out.backward(d)
        res.append([out, xi.grad] + [p.grad for p in blk.parameters()])
    torch.cuda.synchronize()
    for u, v in zip(*res):
        assert torch.equal(u, v)
    assert float(res[0][1].float().abs().max()) > 0


def test_windowed_block_step_replays_from_a_graph(cuda):
    """The DeepSeek-V3 block under an expert window (one rank's share, shared expert included) with
    sync_free_expert_window: forward and backward captured once and replayed on changing inputs,
    each replay bit-identical to an eager twin."""
    graphed = _dsv3_window_block(cuda, True)
    eager = copy.deepcopy(graphed)
    shape = (2, 256, 512)
    gen = torch.Generator().manual_seed(9)
    x_static = torch.randn(shape, generator=gen).to(torch.bfloat16).to(cuda).requires_grad_(True)
    dout_static = torch.randn(shape, generator=gen).to(torch.bfloat16).to(cuda)

    def step(blk, x, dout):
        out = blk(x)
        out.backward(dout)
        return out

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(graphed, x_static, dout_static)
    torch.cuda.current_stream().wait_stream(side)
    graphed.zero_grad(set_to_none=True)
    x_static.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = step(graphed, x_static, dout_static)
    for trial in range(4):
        if trial:
            with torch.no_grad():
                x_static.copy_(torch.randn(shape, generator=gen).to(torch.bfloat16))
                dout_static.copy_(torch.randn(shape, generator=gen).to(torch.bfloat16))
        graph.replay()
        torch.cuda.synchronize()
        eager.zero_grad(set_to_none=True)
        x = x_static.detach().clone().requires_grad_(True)
        out = step(eager, x, dout_static)
        torch.cuda.synchronize()
        assert torch.equal(out_static, out), trial
        assert torch.equal(x_static.grad, x.grad), trial
        want, got = _grads(eager), _grads(graphed)
        assert set(got) == set(want) and len(got) >= 4
        for k in want:
            assert torch.equal(got[k], want[k]), (trial, k)
