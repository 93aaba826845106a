"""Pins the router restatements (oracle/routing.py) against the library calls the reference makes
(torch.softmax, torch.topk) on tie-free rows, their invariants, and a brute-force statement of the
DeepSeek-V3 group-limited selection on a tiny shape."""
import math
import itertools

import pytest
import torch

from oracle import routing as R


@pytest.mark.parametrize("T,N,K,renorm", [(512, 8, 2, True), (2048, 64, 8, False), (256, 256, 8, True)])
def test_olmoe_router_equals_torch_topk_on_tie_free_rows(T, N, K, renorm):
    logits = torch.randn(T, N, generator=torch.Generator().manual_seed(N))
    assert R.min_topk_gap_ulps(torch.softmax(logits, 1), K) > 4.0
    w, e, p = R.olmoe_router(logits, K, renorm, torch.float32)
    tw, te = torch.topk(torch.softmax(logits, dim=1, dtype=torch.float), K, dim=-1)   # moe.py:467-468
    if renorm:
        tw = tw / tw.sum(dim=-1, keepdim=True)
    assert torch.equal(e, te) and torch.equal(w, tw)
    assert bool((w[:, :-1] >= w[:, 1:]).all())
    assert bool((torch.sort(e, 1).values[:, 1:] != torch.sort(e, 1).values[:, :-1]).all())
    if renorm:
        assert torch.allclose(w.sum(1), torch.ones(T), atol=1e-6)


def test_tie_break_is_lowest_index_first():
    logits = torch.zeros(4, 16)
    logits[1, 5:9] = 1.0
    _, e, _ = R.olmoe_router(logits, 3, False, torch.float32)
    assert e[0].tolist() == [0, 1, 2] and e[1].tolist() == [5, 6, 7]


def test_gap_metric_flags_near_ties():
    p = torch.tensor([[0.5, 0.25, 0.25 * (1 + 2 ** -23), 0.0]])
    assert R.min_topk_gap_ulps(p, 2) <= 1.0
    assert R.min_topk_gap_ulps(torch.tensor([[0.5, 0.3, 0.2]]), 2) > 1e5


def _dsv3_brute(scores, bias, n_group, topk_group, K):
    """Direct statement of modeling_deepseek_v3.py:164-180 with python loops."""
    T, N = scores.shape
    gs = N // n_group
    out = []
    for t in range(T):
        c = [float(scores[t, i] + bias[i]) for i in range(N)]
        gsc = []
        for g in range(n_group):
            top2 = sorted(c[g * gs:(g + 1) * gs], reverse=True)[:2]
            gsc.append(sum(top2))
        keep = sorted(range(n_group), key=lambda g: (-gsc[g], g))[:topk_group]
        masked = [c[i] if (i // gs) in keep else 0.0 for i in range(N)]
        out.append(sorted(range(N), key=lambda i: (-masked[i], i))[:K])
    return torch.tensor(out)


def test_dsv3_group_limited_topk_brute_force():
    g = torch.Generator().manual_seed(0)
    scores = torch.rand(200, 16, generator=g)
    bias = torch.randn(16, generator=g) * 0.1
    e, _ = R.dsv3_topk_indices(scores, bias, 4, 2, 2)
    # fp32 sums in the restatement vs python floats here: compare as sets where group scores are
    # not within rounding of each other (always true for this seed)
    assert torch.equal(torch.sort(e, 1).values, torch.sort(_dsv3_brute(scores, bias, 4, 2, 2), 1).values)


def test_dsv3_router_invariants_and_library_topk():
    g = torch.Generator().manual_seed(1)
    T, H, N = 300, 64, 256
    x = torch.randn(T, H, generator=g); W = torch.randn(N, H, generator=g) * 0.06
    bias = torch.randn(N, generator=g) * 0.1
    e, w, logits = R.dsv3_router(x, W, bias, 8, 4, 8, True, 2.5)
    assert torch.allclose(w.sum(1), torch.full((T,), 2.5), atol=1e-5)
    scores = logits.sigmoid()
    # selected experts lie in at most topk_group groups and weights are the un-biased scores
    assert int((e // 32).sort(1).values.diff(dim=1).ne(0).sum(1).max()) + 1 <= 4
    ww = scores.gather(1, e); ww = ww / (ww.sum(-1, keepdim=True) + 1e-20) * 2.5
    assert torch.allclose(w, ww)
    # same sets as the reference's sequence of torch.topk calls (sorted=False there)
    sfc = scores + bias
    group_scores = sfc.view(T, 8, 32).topk(2, dim=-1)[0].sum(dim=-1)
    group_idx = torch.topk(group_scores, k=4, dim=-1, sorted=False)[1]
    mask = torch.zeros_like(group_scores).scatter_(1, group_idx, 1)
    score_mask = mask.unsqueeze(-1).expand(-1, 8, 32).reshape(T, N)
    ref = torch.topk(sfc.masked_fill(~score_mask.bool(), 0.0), k=8, dim=-1, sorted=False)[1]
    assert torch.equal(torch.sort(e, 1).values, torch.sort(ref, 1).values)


# ---- auxiliary load-balancing loss ------------------------------------------------------------
def _brute_force_balance_loss(logits, N, K):
    """Token-by-token statement: c[e] = share of tokens with e among their K most probable experts,
    P[e] = mean probability; loss = N * sum_e c[e] P[e]."""
    T = logits.shape[0]
    c = [0.0] * N; P = [0.0] * N
    for t in range(T):
        row = [float(v) for v in logits[t].double()]
        m = max(row); ex = [math.exp(v - m) for v in row]; z = sum(ex)
        p = [v / z for v in ex]
        order = sorted(range(N), key=lambda i: (-p[i], i))[:K]
        for e in order:
            c[e] += 1.0 / T
        for e in range(N):
            P[e] += p[e] / T
    return N * sum(ci * pi for ci, pi in zip(c, P))


def test_balance_loss_restatement_vs_brute_force():
    g = torch.Generator().manual_seed(3)
    layers = tuple(torch.randn(40, 12, generator=g) for _ in range(3))
    want = _brute_force_balance_loss(torch.cat(layers), 12, 3)
    got = float(R.load_balancing_loss(layers, 12, 3))
    assert abs(got - want) <= 1e-5 * want
    per_layer = sum(_brute_force_balance_loss(l, 12, 3) for l in layers)
    assert abs(float(R.layer_level_load_balancing_loss(layers, 12, 3)) - per_layer) <= 1e-5 * per_layer


def test_balance_loss_closed_forms():
    # every token has the same logits: the K most probable experts get all the tokens
    row = torch.tensor([0.3, 2.0, -1.0, 1.5, 0.0, 0.9])
    p = torch.softmax(row, 0)
    logits = row.expand(50, 6).contiguous()
    want = 6 * float(p[1] + p[3])
    assert abs(float(R.load_balancing_loss((logits,), 6, 2)) - want) < 1e-6
    # perfectly balanced routing with uniform-looking probabilities gives K (the minimum N * K/N * 1/N * N)
    N, K, T = 8, 2, 64
    logits = torch.full((T, N), -10.0)
    for t in range(T):
        logits[t, t % N] = 1.0; logits[t, (t + 1) % N] = 0.5
    loss = float(R.load_balancing_loss((logits,), N, K))
    assert abs(loss - K) < 1e-3


def test_masked_balance_loss_is_the_loss_of_the_kept_tokens():
    """Pins the masked branch of the auxiliary-loss restatement (modeling_olmoe.py:58-83) without
    retyping it: with a 0/1 mask the loss must equal the unmasked loss evaluated on the kept tokens
    alone (every layer's rows filtered by the same mask); an all-ones mask changes nothing; and the
    plausible mistakes — dividing by the token count instead of the mask sum, or masking only one
    of the two factors — give a different value."""
    g = torch.Generator().manual_seed(4)
    B, S, N, K, L = 3, 40, 16, 4, 3
    layers = tuple(torch.randn(B * S, N, generator=g) * 2 for _ in range(L))
    mask = (torch.rand(B, S, generator=g) > 0.35).float()
    assert 0 < int(mask.sum()) < B * S
    keep = mask.reshape(-1).bool()
    want = R.load_balancing_loss(tuple(l[keep] for l in layers), N, K)
    got = R.load_balancing_loss(layers, N, K, attention_mask=mask)
    assert abs(float(got) - float(want)) <= 1e-6 * float(want)
    plain = R.load_balancing_loss(layers, N, K)
    assert abs(float(R.load_balancing_loss(layers, N, K, attention_mask=torch.ones(B, S))) - float(plain)) <= 1e-6 * float(plain)
    assert abs(float(got) - float(plain)) > 1e-4 * float(plain)
    # dividing by the number of tokens instead of the mask sum scales the loss by (sum m / T)^2
    frac = float(mask.mean())
    assert abs(float(got) * frac * frac - float(got)) > 1e-2 * float(got)
    # gradient flows only into kept tokens
    lg = tuple(l.clone().requires_grad_(True) for l in layers)
    R.load_balancing_loss(lg, N, K, attention_mask=mask).backward()
    for l in lg:
        assert float(l.grad[~keep].abs().max()) == 0.0 and float(l.grad[keep].abs().max()) > 0.0
