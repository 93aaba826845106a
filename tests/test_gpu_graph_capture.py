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
