"""om_moe_sort_static — the entry point that allocates nothing (its block table is a fixed device
array inside the library) — against om_moe_sort, both called straight through the C ABI on the same
inputs.  Bar: every output array bit for bit.  Calls come in pairs, the second on a smaller input,
so that whatever the first call left in the array would show if the second depended on it; the
outputs are pre-filled with a sentinel so untouched tails must match as well."""
import pytest
import torch

from util import routed_experts

pytestmark = pytest.mark.gpu


def _outputs(T, K, NR, cuda):
    i32 = dict(dtype=torch.int32, device=cuda)
    return [torch.full((NR + 1,), -7, **i32), torch.full((T + 1,), -7, **i32),
            torch.full((T * K,), -7, **i32), torch.full((T * K,), -7, **i32), torch.full((T * K,), -7, **i32)]


def _both(se, start, end, cuda):
    from optimus import _native as n
    lib = n.lib()
    T, K = se.shape
    NR = end - start
    se = se.to(cuda).contiguous()
    ws_bytes = int(lib.om_moe_sort_workspace_bytes(T, K, NR))
    ws = torch.empty(max(ws_bytes, 4) // 4 + 1, dtype=torch.int32, device=cuda)
    a, b = _outputs(T, K, NR, cuda), _outputs(T, K, NR, cuda)
    n.check(lib.om_moe_sort(n.ptr(se), n.index_code(se), T, K, start, end, *[n.ptr(t) for t in a],
                            n.ptr(ws), ws.numel() * 4, n.stream()), "om_moe_sort")
    n.check(lib.om_moe_sort_static(n.ptr(se), n.index_code(se), T, K, start, end, *[n.ptr(t) for t in b],
                                   n.stream()), "om_moe_sort_static")
    torch.cuda.synchronize()
    return a, b


@pytest.mark.parametrize("first,second", [
    ((16384, 64, 8, 0, 64, 0.0, torch.int64), (512, 64, 8, 0, 64, 1.2, torch.int64)),     # C3 then C4
    ((8192, 256, 8, 64, 96, 0.0, torch.int64), (257, 16, 4, 4, 12, 2.0, torch.int32)),    # C5 window, then tiny
    ((40000, 128, 8, 0, 128, 0.5, torch.int32), (24, 64, 8, 0, 64, 3.0, torch.int64)),
])
def test_static_sort_equals_workspace_sort_twice_in_a_row(cuda, first, second):
    for T, N, K, start, end, skew, dt in (first, second):
        se = routed_experts(T, N, K, seed=T + N + K, skew=skew).to(dt)
        a, b = _both(se, start, end, cuda)
        assert int(a[0][-1]) > 0
        for name, x, y in zip(("cum_token_counts", "cum_expert_counts_ep", "input_indices", "output_indices",
                               "selected_experts_indices"), a, b):
            assert torch.equal(x, y), (name, T, N, K)


def test_static_sort_rejects_what_does_not_fit(cuda):
    from optimus import _native as n
    lib = n.lib()
    cap = int(lib.om_moe_sort_static_capacity_bytes())
    assert cap == 4 << 20
    T, K, NR = 262400, 8, 1024                       # 1025 count blocks x 1024 experts > 1 Mi table cells
    assert int(lib.om_moe_sort_workspace_bytes(T, K, NR)) > cap
    se = torch.zeros((T, K), dtype=torch.int32, device=cuda)
    out = _outputs(T, K, NR, cuda)
    rc = lib.om_moe_sort_static(n.ptr(se), n.OM_I32, T, K, 0, NR, *[n.ptr(t) for t in out], n.stream())
    assert rc == -6 and b"workspace" in lib.om_strerror(rc).lower()
    torch.cuda.synchronize()
    assert all(bool((t == -7).all()) for t in out)   # nothing was launched
    # one table cell under the limit is taken
    T2 = 2048 * 1022 // K
    assert int(lib.om_moe_sort_workspace_bytes(T2, K, NR)) <= cap


def test_static_sort_allocates_nothing_and_replays_from_a_graph(cuda):
    """What the entry point is for: after one call outside any capture (which resolves the array's
    address), further calls leave the device's free memory and torch's allocator untouched, and the
    call can be recorded into a HIP graph; every replay on new inputs gives om_moe_sort's bits."""
    from optimus import _native as n
    lib = n.lib()
    T, N, K, start, end = 4096, 64, 8, 16, 48
    NR = end - start
    se = routed_experts(T, N, K, seed=1).to(cuda).contiguous()
    out = _outputs(T, K, NR, cuda)

    def call():
        n.check(lib.om_moe_sort_static(n.ptr(se), n.index_code(se), T, K, start, end,
                                       *[n.ptr(t) for t in out], n.stream()), "om_moe_sort_static")
    call()                                            # first call: outside capture
    torch.cuda.synchronize()
    free0, alloc0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for trial in range(3):
        se.copy_(routed_experts(T, N, K, seed=10 + trial, skew=0.5 * trial).to(cuda))
        for t in out:
            t.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        want, _ = _both(se.clone(), start, end, cuda)      # eager work between the replays
        for name, x, y in zip(("cum_token_counts", "cum_expert_counts_ep", "input_indices", "output_indices",
                               "selected_experts_indices"), want, out):
            assert torch.equal(x, y), (trial, name)
