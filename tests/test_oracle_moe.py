"""Pins the C restatement of the MoE index / row kernels (oracle/moe_oracle.c) against checks that
do not retype it: closed forms through library routines (stable argsort, bincount, cumsum,
fancy indexing, index_add_), algebraic identities (adjoint), and brute force on tiny inputs.
The reference holds no golden vectors for this path, so these are what fixes the oracle."""
import numpy as np
import pytest
import torch

from oracle import clib
from util import bits, from_bits, routed_experts


def closed_form(se, start, end):
    """Stable counting sort stated with numpy library calls only."""
    T, K = se.shape
    flat = se.reshape(-1)
    local = (flat >= start) & (flat < end)
    j_all = np.nonzero(local)[0]                       # kept (t,k) pairs in row-major order
    keys = flat[j_all] - start
    order = np.argsort(keys, kind="stable")            # position p holds pair j_all[order[p]]
    pos = np.empty_like(order)
    pos[order] = np.arange(order.size)                 # pair index -> sorted position
    cum = np.concatenate([[0], np.cumsum(np.bincount(keys, minlength=end - start))])
    per_token = local.reshape(T, K).sum(1)
    cum_ep = np.concatenate([[0], np.cumsum(per_token)])
    return dict(cum_token_counts=cum.astype(np.int32), cum_expert_counts_ep=cum_ep.astype(np.int32),
                output_indices=pos.astype(np.int32),
                input_indices=(j_all[order] // K).astype(np.int32),
                selected_experts_indices=(j_all % K).astype(np.int32))


@pytest.mark.parametrize("T,N,K,start,end,skew", [
    (8, 4, 2, 0, 4, 0.0), (64, 8, 2, 0, 8, 0.0), (512, 64, 8, 0, 64, 1.2), (2048, 8, 2, 0, 8, 0.0),
    (1024, 256, 8, 64, 96, 0.0), (256, 16, 4, 4, 12, 2.5), (16, 64, 8, 0, 64, 4.0), (4096, 64, 8, 0, 64, 0.0)])
def test_index_construction_is_stable_counting_sort(T, N, K, start, end, skew):
    se = routed_experts(T, N, K, seed=T * 7 + K, skew=skew).numpy()
    got = clib.index_construction(se, end - start, start, end)
    want = closed_form(se, start, end)
    for k, v in want.items():
        assert np.array_equal(got[k], v), k
    # the result does not depend on the tokens-per-thread blocking of the reference kernels
    for tb in (1, 2, 4):
        if T % tb == 0:
            alt = clib.index_construction(se, end - start, start, end, tokens_per_thread=tb)
            for k in want:
                assert np.array_equal(alt[k], got[k]), (k, tb)


def test_index_construction_brute_force_tiny():
    """Every routing of 3 tokens x top-2 over 3 experts: rows grouped by expert, token order kept."""
    import itertools
    pairs = [p for p in itertools.permutations(range(3), 2)]
    for combo in itertools.product(pairs, repeat=3):
        se = np.array(combo, dtype=np.int64)
        se8 = np.concatenate([se, np.tile(se[:1], (5, 1))])   # pad to T=8 (T % 8 == 0)
        got = clib.index_construction(se8, 3, 0, 3)
        rows = [(int(se8[t, k]), t, k) for t in range(8) for k in range(2)]
        rows_sorted = sorted(rows, key=lambda r: (r[0], r[1]))     # expert, then token
        assert [r[1] for r in rows_sorted] == got["input_indices"].tolist()
        for j, (e, t, k) in enumerate(rows):
            p = got["output_indices"][j]
            assert rows_sorted[p] == (e, t, k) and got["selected_experts_indices"][j] == k


def _case(dtype, T=96, N=8, K=2, E=40, start=0, end=8, seed=0):
    se = routed_experts(T, N, K, seed=seed + 5).numpy()
    idx = clib.index_construction(se, end - start, start, end)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, E, generator=g).to(dtype)
    y = torch.randn(idx["num_routed_tokens"], E, generator=g).to(dtype)
    w = torch.rand(T, K, generator=g).to(dtype)
    d = torch.randn(T, E, generator=g).to(dtype)
    return se, idx, x, y, w, d


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("start,end", [(0, 8), (2, 6)])
def test_row_kernels_against_library_expressions(dtype, start, end):
    se, idx, x, y, w, d = _case(dtype, start=start, end=end)
    T, K = w.shape
    ii = torch.from_numpy(idx["input_indices"]).long()
    oi = torch.from_numpy(idx["output_indices"]).long()
    si = torch.from_numpy(idx["selected_experts_indices"]).long()
    # gather = fancy indexing (moe.py:237)
    assert np.array_equal(clib.index_gather(bits(x), idx["input_indices"]), bits(x[ii]))
    # token of every routed pair, from the permutation itself
    tok = ii[oi]
    # scatter-reduce = index_add_ of the un-permuted rows in fp32, one rounding (moe.py:273-281)
    want = torch.zeros(T, y.shape[1]).index_add_(0, tok, y.float()[oi]).to(dtype)
    got = from_bits(clib.shuffle_sub_matrix_reduce(bits(y), idx["cum_expert_counts_ep"], idx["output_indices"], T), dtype)
    assert torch.allclose(got.float(), want.float(), rtol=0, atol=1e-6 if dtype == torch.float32 else 4e-2)
    # weighted combine (moe.py:313-325)
    scale = w.float()[tok, si]
    want = torch.zeros(T, y.shape[1]).index_add_(0, tok, y.float()[oi] * scale[:, None]).to(dtype)
    got = from_bits(clib.reduce_ggemm_output(bits(y), bits(w), idx["cum_expert_counts_ep"],
                                            idx["selected_experts_indices"], idx["output_indices"]), dtype)
    assert torch.allclose(got.float(), want.float(), rtol=0, atol=1e-5 if dtype == torch.float32 else 4e-2)
    # backward (moe.py:365-376): dy[pos] = w * dout[t];  dw[t,k] = <y[pos], dout[t]>
    dy, dw = clib.reduce_ggemm_output_backward(bits(d), bits(y), bits(w), idx["selected_experts_indices"],
                                               idx["input_indices"], idx["output_indices"])
    dy = from_bits(dy, dtype); dw = from_bits(dw, dtype)
    want_dy = torch.zeros_like(y.float())
    want_dy[oi] = scale[:, None] * d.float()[tok]
    assert torch.allclose(dy.float(), want_dy.to(dtype).float(), rtol=0, atol=1e-6 if dtype == torch.float32 else 2e-2)
    want_dw = torch.zeros(T, K)
    want_dw[tok, si] = (y.float()[oi] * d.float()[tok]).sum(1)
    tol = 1e-4 if dtype == torch.float32 else 6e-2
    assert torch.allclose(dw.float(), want_dw, rtol=tol, atol=tol)


def test_combine_adjoint_identity():
    """<combine(y), d> == <y, combine^T(d)> and <combine(y; w), d> is linear in w with gradient dw."""
    se, idx, x, y, w, d = _case(torch.float32, T=64, E=24)
    out = torch.from_numpy(clib.reduce_ggemm_output(bits(y), bits(w), idx["cum_expert_counts_ep"],
                                                    idx["selected_experts_indices"], idx["output_indices"]))
    dy, dw = clib.reduce_ggemm_output_backward(bits(d), bits(y), bits(w), idx["selected_experts_indices"],
                                               idx["input_indices"], idx["output_indices"])
    lhs = float((out.double() * d.double()).sum())
    assert abs(lhs - float((y.double() * torch.from_numpy(dy).double()).sum())) <= 1e-4 * abs(lhs)
    assert abs(lhs - float((w.double() * torch.from_numpy(dw).double()).sum())) <= 1e-4 * abs(lhs)
    # gather / scatter-reduce are adjoint too
    gx = torch.from_numpy(clib.index_gather(bits(x), idx["input_indices"]))
    sy = torch.from_numpy(clib.shuffle_sub_matrix_reduce(bits(y), idx["cum_expert_counts_ep"], idx["output_indices"], x.shape[0]))
    a = float((gx.double() * y.double()).sum()); b = float((x.double() * sy.double()).sum())
    assert abs(a - b) <= 1e-4 * abs(a)


def test_index_add_serial_semantics():
    g = torch.Generator().manual_seed(1)
    inp = torch.randn(50, 12, generator=g); base = torch.randn(9, 12, generator=g)
    idx = torch.randint(0, 9, (50,), generator=g).to(torch.int32)
    out = base.numpy().copy()
    clib.index_add(inp.numpy(), out, idx.numpy())
    assert np.allclose(out, base.index_add(0, idx.long(), inp).numpy(), atol=1e-5)


def test_swiglu_glue_against_autograd():
    g = torch.Generator().manual_seed(2)
    a = torch.randn(1000, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(1000, generator=g, dtype=torch.float64, requires_grad=True)
    dh = torch.randn(1000, generator=g, dtype=torch.float64)
    h = torch.nn.functional.silu(a) * b
    h.backward(dh)
    assert np.allclose(clib.swiglu_fwd(a.detach().float().numpy(), b.detach().float().numpy()), h.detach().numpy(), atol=1e-5)
    dg, du = clib.swiglu_bwd(dh.float().numpy(), a.detach().float().numpy(), b.detach().float().numpy())
    assert np.allclose(dg, a.grad.numpy(), atol=1e-5) and np.allclose(du, b.grad.numpy(), atol=1e-5)


def test_bf16_rounding_rule():
    x = torch.randn(100000, generator=torch.Generator().manual_seed(3)) * 37.0
    x[:4] = torch.tensor([0.0, -0.0, float("inf"), 1.00390625])   # last: exact tie -> even
    assert np.array_equal(clib.f32_to_bf16_bits(x.numpy()), bits(x.to(torch.bfloat16)))


def test_layer_restatements_agree_on_tiny_shapes():
    """The per-expert loop (slow block), the K1..K6 restatement and the token-by-token textbook
    formula are three independent evaluations of one function."""
    from oracle import moe_layer as L, routing as R
    torch.manual_seed(0)
    T, H, N, K, I = 64, 32, 8, 2, 48
    x = torch.randn(T, H); Wg = torch.randn(N, H) * 0.3
    wg = torch.randn(N, I, H) * 0.1; wu = torch.randn(N, I, H) * 0.1; wd = torch.randn(N, H, I) * 0.1
    for renorm in (True, False):
        out, logits = L.olmoe_slow_block(x, Wg, wg, wu, wd, K, renorm)
        w, e, _ = R.olmoe_router(logits, K, renorm, torch.float32)
        fast, _ = L.fast_block_restatement(x, w, e, wg, wu, wd)
        dense = L.dense_formula(x, w, e, wg, wu, wd)
        assert torch.allclose(out, fast, atol=1e-5) and torch.allclose(out, dense, atol=1e-5)
    # expert window: the windowed blocks of all ranks sum to the full block
    parts = []
    for s in (0, 4):
        f, _ = L.fast_block_restatement(x, w, e, wg[s:s + 4], wu[s:s + 4], wd[s:s + 4], expert_start_idx=s)
        parts.append(f)
    assert torch.allclose(parts[0] + parts[1], fast, atol=1e-5)


def _dsv3_tiny(seed=3):
    """A DeepSeek-V3-shaped toy: 16 experts in 4 groups, 2 groups kept, top-4, one shared expert."""
    g = torch.Generator().manual_seed(seed)
    T, H, N, I = 40, 24, 16, 20
    x = torch.randn(T, H, generator=g)
    Wr = torch.randn(N, H, generator=g) * 0.3
    bias = torch.randn(N, generator=g) * 0.1
    wg = torch.randn(N, I, H, generator=g) * 0.2
    wu = torch.randn(N, I, H, generator=g) * 0.2
    wd = torch.randn(N, H, I, generator=g) * 0.2
    sg = torch.randn(I, H, generator=g) * 0.2
    su = torch.randn(I, H, generator=g) * 0.2
    sd = torch.randn(H, I, generator=g) * 0.2
    return dict(x=x, Wr=Wr, bias=bias, wg=wg, wu=wu, wd=wd, sg=sg, su=su, sd=sd,
                route=dict(n_group=4, topk_group=2, top_k=4, norm_topk_prob=True,
                           routed_scaling_factor=2.5))


def _dsv3_block(c, start=0, count=None, shared=True, tensors=None):
    from oracle import moe_layer as L
    t = tensors or c
    count = c["wg"].shape[0] if count is None else count
    sl = slice(start, start + count)
    zero = torch.zeros_like
    ws = (t["sg"], t["su"], t["sd"]) if shared else (zero(t["sg"]), zero(t["su"]), zero(t["sd"]))
    return L.dsv3_moe_block(t["x"], t["Wr"], t["bias"], t["wg"][sl], t["wu"][sl], t["wd"][sl], *ws,
                            expert_start_idx=start, **c["route"])


def test_dsv3_block_is_dense_formula_plus_shared_expert():
    """Pins oracle.moe_layer.dsv3_moe_block (modeling_deepseek_v3.py:221-275) on a tiny shape against
    evaluations that share none of its code: the token-by-token textbook sum over the routed experts
    (weights and ids from the brute-force-pinned router) plus the shared expert's MLP on every
    token.  Deliberately wrong variants (no shared expert, a window offset by one expert, weights
    taken from the biased scores) must fail the same comparison."""
    from oracle import moe_layer as L, routing as R
    c = _dsv3_tiny()
    out, ids, w = _dsv3_block(c)
    ids_r, w_r, _ = R.dsv3_router(c["x"], c["Wr"], c["bias"], **c["route"])
    assert torch.equal(ids, ids_r) and torch.equal(w, w_r)
    # router invariants that fix its meaning: K distinct experts, from at most topk_group groups,
    # weights sum to the scaling factor
    assert all(len(set(r.tolist())) == 4 for r in ids)
    assert all(len({int(e) // 4 for e in r}) <= 2 for r in ids)
    assert torch.allclose(w.sum(1), torch.full((w.shape[0],), 2.5), atol=1e-5)
    routed = L.dense_formula(c["x"], w, ids, c["wg"], c["wu"], c["wd"])
    shared = L.expert_mlp(c["x"], c["sg"], c["su"], c["sd"])
    assert torch.allclose(out, routed + shared, atol=2e-5)
    scale = float(out.abs().mean())
    # a block without its shared expert is a different function
    assert float((out - routed).abs().mean()) > 0.05 * scale
    # so is one whose window is offset by one expert (weights of expert e+1 used for id e) ...
    shifted = L.dense_formula(c["x"], w, ids, c["wg"].roll(1, 0), c["wu"].roll(1, 0), c["wd"].roll(1, 0))
    assert float((out - shifted - shared).abs().mean()) > 0.05 * scale
    # ... and one whose weights come from sigmoid + bias instead of the plain sigmoid (:187)
    s = torch.sigmoid(torch.nn.functional.linear(c["x"], c["Wr"]))
    wb = (s + c["bias"]).gather(1, ids)
    wb = wb / (wb.sum(1, keepdim=True) + 1e-20) * 2.5
    biased = L.dense_formula(c["x"], wb, ids, c["wg"], c["wu"], c["wd"])
    assert float((out - biased - shared).abs().mean()) > 1e-3 * scale


def test_dsv3_block_windows_sum_to_the_whole_block():
    """Expert parallelism of the DeepSeek-V3 block (modeling_deepseek_v3.py:226-229): each rank adds
    only its window's experts, so the routed parts of all ranks' blocks sum to the EP=1 routed part,
    and a window that owns no selected expert contributes exactly the shared expert."""
    from oracle import moe_layer as L
    c = _dsv3_tiny(seed=4)
    full, ids, _ = _dsv3_block(c, shared=False)
    parts = [_dsv3_block(c, start=s, count=4, shared=False)[0] for s in (0, 4, 8, 12)]
    assert torch.allclose(sum(parts), full, atol=2e-5)
    # every window is a strict part (none is empty, none is everything) for this fixture
    assert all(0.0 < float(p.abs().sum()) < float(full.abs().sum()) for p in parts)
    # a window's block only sees tokens that chose one of its experts
    for s, p in zip((0, 4, 8, 12), parts):
        hit = ((ids >= s) & (ids < s + 4)).any(1)
        assert torch.equal(p[~hit], torch.zeros_like(p[~hit]))
        assert bool((p[hit].abs().sum(1) > 0).all())
    with_shared = _dsv3_block(c, start=4, count=4, shared=True)[0]
    assert torch.allclose(with_shared - parts[1], L.expert_mlp(c["x"], c["sg"], c["su"], c["sd"]), atol=2e-5)


def test_dsv3_block_gradients_match_the_dense_formula():
    """Backward of the DeepSeek-V3 block restatement: autograd through the per-expert index_add_
    loop against autograd through the token-by-token formula (separate graphs), for the input,
    the router weight (reached only through the gathered sigmoid scores: the index selection is
    no_grad and the bias gets no gradient, modeling_deepseek_v3.py:186-187) and the experts."""
    from oracle import moe_layer as L, routing as R
    c = _dsv3_tiny(seed=5)
    names = ("x", "Wr", "wg", "wu", "wd", "sg", "su", "sd")
    d = torch.randn(c["x"].shape, generator=torch.Generator().manual_seed(9))

    a = {k: (v.clone().requires_grad_(True) if k in names else v) for k, v in c.items()}
    a["bias"] = c["bias"].clone().requires_grad_(True)
    out, ids, w = _dsv3_block(c, tensors=a)
    out.backward(d)
    assert a["bias"].grad is None

    b = {k: (v.clone().requires_grad_(True) if k in names else v) for k, v in c.items()}
    ids_b, w_b, _ = R.dsv3_router(b["x"], b["Wr"], b["bias"], **c["route"])
    ref = L.dense_formula(b["x"], w_b, ids_b, b["wg"], b["wu"], b["wd"]) + \
        L.expert_mlp(b["x"], b["sg"], b["su"], b["sd"])
    ref.backward(d)
    for k in names:
        assert torch.allclose(a[k].grad, b[k].grad, rtol=1e-4, atol=1e-5), k
    # the routing weights do carry gradient into the router weight
    assert float(a["Wr"].grad.abs().sum()) > 0


def test_fast_block_sequence_is_the_layer_and_its_gradients():
    """fast_block_sequence (gather, three segment products, silu, multiply, combine, and autograd
    through them) in float32 equals the token-by-token textbook formula and ITS autograd gradients,
    with and without an expert window; in bfloat16 it is the same function up to bf16 roundings and
    returns bf16 gradients for every input."""
    from oracle import moe_layer as L, routing as R
    torch.manual_seed(5)
    T, H, N, K, I = 48, 32, 8, 3, 40
    x = torch.randn(T, H); Wg = torch.randn(N, H) * 0.3
    wg = torch.randn(N, I, H) * 0.1; wu = torch.randn(N, I, H) * 0.1; wd = torch.randn(N, H, I) * 0.1
    d = torch.randn(T, H)
    w, e, _ = R.olmoe_router(x @ Wg.t(), K, False, torch.float32)
    for start, count in ((0, N), (2, 4)):
        sl = slice(start, start + count)
        leaf = {k: v.clone().requires_grad_(True) for k, v in dict(x=x, w=w, wg=wg[sl], wu=wu[sl], wd=wd[sl]).items()}
        dense = L.dense_formula(leaf["x"], leaf["w"], e, leaf["wg"], leaf["wu"], leaf["wd"], expert_start_idx=start)
        dense.backward(d)
        out, grads = L.fast_block_sequence(x, w, e, wg[sl], wu[sl], wd[sl], d, expert_start_idx=start)
        assert torch.allclose(out, dense, atol=1e-5)
        for a, b in (("x", "x"), ("routing_weights", "w"), ("w_gate", "wg"), ("w_up", "wu"), ("w_down", "wd")):
            assert torch.allclose(grads[a], leaf[b].grad, atol=2e-5), a
    bf = torch.bfloat16
    out16, g16 = L.fast_block_sequence(x.to(bf), w.to(bf), e, wg.to(bf), wu.to(bf), wd.to(bf), d.to(bf))
    out32, g32 = L.fast_block_sequence(x.to(bf).float(), w.to(bf).float(), e, wg.to(bf).float(), wu.to(bf).float(),
                                       wd.to(bf).float(), d.to(bf).float())
    assert out16.dtype == bf and all(v.dtype == bf for v in g16.values())
    rel = lambda a, b: float((a.float() - b).abs().mean() / b.abs().mean())
    assert 1e-3 < rel(out16, out32) < 1e-2                   # rounded, but only rounded
    for k in g32:
        assert 1e-3 < rel(g16[k], g32[k]) < 1.5e-2, k
