"""Grouped expert GEMMs through optimus.models.common.moe (-> C-ABI om_grouped_gemm_*,
om_merged_mlp_*) against per-expert torch.matmul in fp32 on the same bf16 inputs — the special
case the reference itself uses as its check (optimus/kernels/grouped_linear_forward.py:104-112,
moe.py:174-178).  Bar: a product's output is ONE bf16 rounding of an fp32-accumulated sum, so its
distance from the fp32 reference must be that of the ideally rounded reference (mean_rel 1.41e-3
for Gaussian results) plus fp32 summation-order noise: util.assert_bf16_parity with an excess
factor just above 1 (ONE_ROUNDING), and max-abs <= 2e-2 of the largest magnitude.  The merged MLP
rounds g, u, h (and y) on the way like the reference, hence the wider MLP_BARS."""
import numpy as np
import pytest
import torch

from util import assert_bf16_parity, max_abs, mean_rel

# (excess over the bf16 floor, absolute cap on mean_rel); measured: single products 1.00 x the floor,
# the merged MLP 1.6 x (y) and 1.5-2.5 x (gradients)
ONE_ROUNDING = (1.03, 1.8e-3)
MLP_BARS = {"out": (1.9, 2.7e-3), "grad": (2.9, 4.1e-3)}

pytestmark = pytest.mark.gpu


def _counts(kind, G, rows, seed=0):
    g = torch.Generator().manual_seed(seed)
    if kind == "uniform":
        c = torch.full((G,), rows // G)
        c[: rows - int(c.sum())] += 1
    elif kind == "ragged":
        p = torch.rand(G, generator=g) ** 3
        c = torch.floor(p / p.sum() * rows).long()
        c[0] += rows - int(c.sum())
    elif kind == "empties":
        c = torch.zeros(G, dtype=torch.long)
        hot = torch.randperm(G, generator=g)[: max(1, G // 4)]
        c[hot] = rows // len(hot)
        c[hot[0]] += rows - int(c.sum())
    elif kind == "onehot":   # every row belongs to one expert in the middle
        c = torch.zeros(G, dtype=torch.long)
        c[G // 2] = rows
    cum = torch.zeros(G + 1, dtype=torch.int32)
    cum[1:] = torch.cumsum(c, 0)
    return cum


def _ref_fwd(x, w, cum):
    out = torch.zeros(x.shape[0], w.shape[1])
    for g in range(w.shape[0]):
        s, e = int(cum[g]), int(cum[g + 1])
        out[s:e] = x[s:e].float() @ w[g].float().t()
    return out


CASES = [# few rows per expert with extents that are multiples of 256 (skewed small batches): most tiles hold
         # a handful of valid rows; one expert with many row tiles among empty ones
         ("ragged", 64, 4096, 1024, 2048), ("empties", 64, 3000, 256, 512), ("onehot", 16, 1000, 256, 256),
         ("uniform", 20, 640, 512, 256), ("ragged", 300, 9000, 256, 256), ("ragged", 512, 4097, 256, 512),
         ("uniform", 4, 512, 256, 128), ("ragged", 8, 1000, 256, 512), ("empties", 16, 777, 128, 256),
         ("ragged", 64, 4096, 1024, 2048), ("uniform", 1, 300, 256, 256), ("ragged", 3, 5, 128, 128),
         # several tiles per persistent block, on both tile shapes, with empty experts in between
         ("ragged", 8, 20000, 512, 768), ("ragged", 8, 20000, 384, 640), ("empties", 32, 9000, 512, 1024),
         # more experts than lanes in a wavefront: the per-block tile table is built in several
         # rounds with a carry, the last one partial
         ("ragged", 150, 6000, 128, 128), ("empties", 200, 70000, 256, 256),
         # all the work in one expert: the weight gradient's work-balanced split of the tiles over the
         # XCDs then cuts that expert's tiles eight ways and the zero tiles of the others ride along
         ("onehot", 70, 5000, 256, 512), ("onehot", 9, 3000, 512, 256), ("onehot", 2, 130, 128, 128),
         # extents that are multiples of 64 but not of 128: partial last tiles along the output columns
         # (and, for the weight gradient, along both extents of dW), odd numbers of contraction steps
         ("ragged", 8, 1000, 320, 192), ("uniform", 4, 512, 64, 64), ("empties", 16, 777, 192, 448),
         ("ragged", 64, 20000, 320, 2048), ("onehot", 5, 700, 2048, 320),
         # extents that are multiples of 8 only: partial 16-byte-chunk column masks in the last tile, a
         # last contraction step with fewer than 64 indices (zero-filled in LDS), tiny extents
         ("ragged", 8, 1000, 200, 136), ("uniform", 4, 512, 72, 40), ("empties", 16, 777, 8, 8),
         ("ragged", 6, 900, 328, 1000), ("onehot", 5, 700, 1000, 328), ("ragged", 3, 50, 24, 264)]


@pytest.mark.parametrize("kind,G,rows,N,K", CASES)
def test_grouped_gemm_fwd_dgrad_wgrad(cuda, kind, G, rows, N, K):
    from optimus.models.common.moe import GroupedGemmFunction
    g = torch.Generator().manual_seed(rows)
    x = torch.randn(rows, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(G, N, K, generator=g) * 0.05).to(torch.bfloat16)
    dout = torch.randn(rows, N, generator=g).to(torch.bfloat16)
    cum = _counts(kind, G, rows)
    xd = x.to(cuda).requires_grad_(True)
    wd = w.to(cuda).requires_grad_(True)
    # the reference passes a CPU int32 tensor of offsets and max_tokens_per_expert (moe.py:397-398)
    out = GroupedGemmFunction.apply(xd, wd, cum, int((cum[1:] - cum[:-1]).max()), False)
    out.backward(dout.to(cuda))
    ref = _ref_fwd(x, w, cum)
    assert max_abs(out.float().cpu(), ref) <= 2e-2 * max(1.0, float(ref.abs().max()))
    tag = f"ggemm[{kind},{G},{rows},{N},{K}]"
    assert_bf16_parity(out, ref, *ONE_ROUNDING, tag=tag + " fwd")
    dx_ref = torch.zeros(rows, K); dw_ref = torch.zeros(G, N, K)
    for e in range(G):
        s, t = int(cum[e]), int(cum[e + 1])
        dx_ref[s:t] = dout[s:t].float() @ w[e].float()
        dw_ref[e] = dout[s:t].float().t() @ x[s:t].float()
    assert_bf16_parity(xd.grad, dx_ref, *ONE_ROUNDING, tag=tag + " dgrad")
    assert_bf16_parity(wd.grad, dw_ref, *ONE_ROUNDING, tag=tag + " wgrad")
    assert max_abs(wd.grad.float().cpu(), dw_ref) <= 1e-2 * max(1.0, float(dw_ref.abs().max()))
    # experts without rows get exactly zero weight gradient
    empty = (cum[1:] == cum[:-1])
    if empty.any():
        assert float(wd.grad[empty.to(cuda)].abs().max()) == 0.0


@pytest.mark.parametrize("kind,G,rows,I,H", [("uniform", 4, 512, 128, 256), ("ragged", 8, 1500, 512, 256),
                                            # skewed small batches: a few rows per expert
                                            ("ragged", 64, 4096, 1024, 2048), ("empties", 32, 700, 256, 512),
                                            ("onehot", 8, 500, 128, 256), ("ragged", 40, 1000, 384, 256),
                                            ("empties", 64, 4096, 1024, 2048), ("ragged", 2, 7, 128, 128),
                                            # hidden / ffn sizes that are multiples of 64 only
                                            ("ragged", 8, 1500, 192, 320), ("uniform", 4, 300, 64, 64),
                                            ("empties", 16, 9000, 320, 1088),
                                            # ... and of 8 only
                                            ("ragged", 8, 1500, 200, 328), ("uniform", 4, 300, 8, 8),
                                            ("empties", 16, 2000, 72, 1000), ("ragged", 5, 600, 1000, 72)])
def test_merged_mlp_fused(cuda, kind, G, rows, I, H):
    """MergedMLP (fused gate+up+SwiGLU, fused down-dgrad+SwiGLU-backward, dual dgrad) against the
    fp32 composition silu(x Wg^T) * (x Wu^T) Wd^T under autograd."""
    from optimus.models.common.moe import MergedMLPFunction
    g = torch.Generator().manual_seed(rows + 1)
    x = torch.randn(rows, H, generator=g).to(torch.bfloat16)
    wg = (torch.randn(G, I, H, generator=g) * 0.05).to(torch.bfloat16)
    wu = (torch.randn(G, I, H, generator=g) * 0.05).to(torch.bfloat16)
    wd = (torch.randn(G, H, I, generator=g) * 0.05).to(torch.bfloat16)
    dy = torch.randn(rows, H, generator=g).to(torch.bfloat16)
    cum = _counts(kind, G, rows)
    dev = [t.to(cuda).requires_grad_(True) for t in (x, wg, wu, wd)]
    y = MergedMLPFunction.apply(*dev, cum.to(cuda))
    y.backward(dy.to(cuda))
    ref = [t.float().requires_grad_(True) for t in (x, wg, wu, wd)]
    outs = []
    for e in range(G):
        s, t = int(cum[e]), int(cum[e + 1])
        xe = ref[0][s:t]
        outs.append((torch.nn.functional.silu(xe @ ref[1][e].t()) * (xe @ ref[2][e].t())) @ ref[3][e].t())
    yr = torch.cat(outs)
    yr.backward(dy.float())
    tag = f"merged_mlp[{kind},{G},{rows},{I},{H}]"
    assert_bf16_parity(y, yr, *MLP_BARS["out"], tag=tag + " y")
    assert max_abs(y.float().cpu(), yr.detach()) <= 2e-2 * max(1.0, float(yr.detach().abs().max()))
    for name, a, b in zip(("dx", "dwg", "dwu", "dwd"), dev, ref):
        assert_bf16_parity(a.grad, b.grad, *MLP_BARS["grad"], tag=f"{tag} {name}")


@pytest.mark.parametrize("T,K,N,start,end,I,H,skew", [
    (4096, 8, 64, 0, 64, 512, 512, 0.0),      # 256x256 tiles, forward and weight gradient
    (512, 2, 8, 0, 8, 128, 384, 0.0),         # 128x128 tiles
    (3000, 4, 16, 4, 12, 256, 256, 1.5),      # expert window: only part of the pairs is routed; skew
    (70, 8, 64, 0, 64, 128, 128, 3.0),        # most experts empty, a few rows each
    (16384, 8, 64, 0, 64, 1024, 2048, 0.0),   # C3
])
def test_gathered_merged_mlp_is_bit_identical(cuda, T, K, N, start, end, I, H, skew):
    """The token gather folded into the GEMM loads (om_merged_mlp_gate_up_fwd_gathered,
    om_grouped_gemm_wgrad_gathered) against gather-then-GEMM (om_index_gather + the plain entry
    points): the same products are summed in the same order, so outputs and every gradient must be
    equal bit for bit."""
    from optimus.models.common.moe import (GatheredMergedMLPFunction, MergedMLPFunction,
                                           PrepareInputForGroupGemmFunction, build_token_permutation)
    from util import routed_experts
    G = end - start
    g = torch.Generator().manual_seed(T + I)
    se = routed_experts(T, N, K, seed=T + K, skew=skew).to(cuda)
    cum, cum_ep, ii, oi, _ = build_token_permutation(se, start, end)
    rows = int(cum[-1].item())
    ii, oi = ii[:rows], oi[:rows]
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ws = [(torch.randn(G, I, H, generator=g) * 0.05).to(torch.bfloat16),
          (torch.randn(G, I, H, generator=g) * 0.05).to(torch.bfloat16),
          (torch.randn(G, H, I, generator=g) * 0.05).to(torch.bfloat16)]
    dy = torch.randn(rows, H, generator=g).to(torch.bfloat16).to(cuda)
    results = []
    for gathered in (False, True):
        xd = x.to(cuda).requires_grad_(True)
        wd = [w.to(cuda).requires_grad_(True) for w in ws]
        if gathered:
            y = GatheredMergedMLPFunction.apply(xd, ii, cum_ep, oi, *wd, cum)
        else:
            y = MergedMLPFunction.apply(PrepareInputForGroupGemmFunction.apply(xd, ii, cum_ep, oi), *wd, cum)
        y.backward(dy)
        results.append([y.detach(), xd.grad] + [w.grad for w in wd])
    for name, a, b in zip(("y", "dx", "dw_gate", "dw_up", "dw_down"), *results):
        assert torch.equal(a, b), name
    assert results[0][0].shape == (rows, H) and bool(torch.isfinite(results[1][0].float()).all())


def test_gathered_merged_mlp_with_no_routed_rows(cuda):
    """An expert window that receives no token: empty output, zero weight gradients, zero input
    gradient, no launch on empty index arrays."""
    from optimus.models.common.moe import GatheredMergedMLPFunction, build_token_permutation
    T, K, H, I, G = 64, 2, 128, 128, 2
    se = torch.zeros(T, K, dtype=torch.int64, device=cuda)
    se[:, 1] = 1                                     # every token picks experts 0 and 1
    cum, cum_ep, ii, oi, _ = build_token_permutation(se, 4, 6)   # window [4, 6): nothing routed
    assert int(cum[-1].item()) == 0
    x = torch.randn(T, H, device=cuda).to(torch.bfloat16).requires_grad_(True)
    ws = [torch.randn(G, I, H, device=cuda).to(torch.bfloat16).requires_grad_(True),
          torch.randn(G, I, H, device=cuda).to(torch.bfloat16).requires_grad_(True),
          torch.randn(G, H, I, device=cuda).to(torch.bfloat16).requires_grad_(True)]
    y = GatheredMergedMLPFunction.apply(x, ii[:0], cum_ep, oi[:0], *ws, cum)
    assert y.shape == (0, H)
    y.sum().backward()
    assert float(x.grad.abs().max()) == 0.0
    for w in ws:
        assert float(w.grad.abs().max()) == 0.0


@pytest.mark.parametrize("kind,G,rows,N,K", [("uniform", 4, 512, 256, 128), ("ragged", 8, 1000, 192, 320),
                                            ("empties", 16, 777, 64, 64), ("ragged", 3, 5, 128, 64),
                                            ("uniform", 8, 4096, 512, 256),
                                            # extents that are multiples of 8 only
                                            ("ragged", 8, 1000, 200, 136), ("uniform", 4, 300, 8, 8),
                                            ("empties", 6, 500, 72, 328)])
def test_grouped_gemm_float32(cuda, kind, G, rows, N, K):
    """float32 modules (the reference's GroupedGemmFunction runs in the module's dtype): the fp32
    kernels against per-expert matmul in float64.  fp32 products and sums, so only the order of
    summation differs from torch's fp32 matmul: errors of a few fp32 roundings of the absolute sum."""
    from optimus.models.common.moe import GroupedGemmFunction
    g = torch.Generator().manual_seed(rows + 7)
    x = torch.randn(rows, K, generator=g)
    w = torch.randn(G, N, K, generator=g) * 0.05
    dout = torch.randn(rows, N, generator=g)
    cum = _counts(kind, G, rows)
    xd = x.to(cuda).requires_grad_(True)
    wd = w.to(cuda).requires_grad_(True)
    out = GroupedGemmFunction.apply(xd, wd, cum, int((cum[1:] - cum[:-1]).max()), False)
    assert out.dtype == torch.float32
    out.backward(dout.to(cuda))
    X, W, D = x.double(), w.double(), dout.double()
    ref = torch.zeros(rows, N, dtype=torch.float64)
    dx_ref = torch.zeros(rows, K, dtype=torch.float64)
    dw_ref = torch.zeros(G, N, K, dtype=torch.float64)
    ref_abs, dx_abs, dw_abs = torch.zeros_like(ref), torch.zeros_like(dx_ref), torch.zeros_like(dw_ref)
    for e in range(G):
        s, t = int(cum[e]), int(cum[e + 1])
        ref[s:t] = X[s:t] @ W[e].t(); ref_abs[s:t] = X[s:t].abs() @ W[e].abs().t()
        dx_ref[s:t] = D[s:t] @ W[e]; dx_abs[s:t] = D[s:t].abs() @ W[e].abs()
        dw_ref[e] = D[s:t].t() @ X[s:t]; dw_abs[e] = D[s:t].abs().t() @ X[s:t].abs()
    for name, got, want, scale in (("out", out, ref, ref_abs), ("dx", xd.grad, dx_ref, dx_abs),
                                   ("dw", wd.grad, dw_ref, dw_abs)):
        err = (got.detach().double().cpu() - want).abs()
        assert bool((err <= 2e-6 * scale + 1e-30).all()), (name, float((err / (scale + 1e-30)).max()))
    empty = (cum[1:] == cum[:-1])
    if empty.any():
        assert float(wd.grad[empty.to(cuda)].abs().max()) == 0.0


# sizes of the seeded sweeps: multiples of 128, and multiples of 8 only (partial last tiles along every
# extent, a last contraction step with 8 to 56 indices)
SWEEP_SIZES = {"multiples_of_128": ([128, 256, 384, 512, 1024], [128, 256, 384, 640, 1024]),
               "multiples_of_8": ([8, 24, 72, 136, 200, 264, 328, 520, 1000], [8, 40, 72, 136, 200, 264, 328, 584, 1000])}


@pytest.mark.parametrize("sizes", sorted(SWEEP_SIZES))
@pytest.mark.parametrize("seed", list(range(24)))
def test_grouped_gemm_random_shapes(cuda, seed, sizes):
    """Seeded sweep over expert counts, row counts and sizes: exercises the persistent-block
    partition (fewer tiles than blocks, remainders over the 8 XCDs, experts without rows, one or many
    tiles per expert) on both tile shapes, against per-expert fp32 matmul."""
    from optimus.models.common.moe import GroupedGemmFunction
    rng = np.random.RandomState(1234 + seed)
    G = int(rng.choice([1, 2, 3, 7, 16, 33, 64, 70]))
    rows = int(rng.choice([1, 17, 255, 256, 257, 1000, 3333, 6000, 20000]))
    N = int(rng.choice(SWEEP_SIZES[sizes][0]))
    K = int(rng.choice(SWEEP_SIZES[sizes][1]))
    kind = ["uniform", "ragged", "empties"][seed % 3]
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(G, N, K, generator=g) * 0.05).to(torch.bfloat16)
    dout = torch.randn(rows, N, generator=g).to(torch.bfloat16)
    cum = _counts(kind, G, rows, seed=seed)
    assert int(cum[-1]) == rows
    xd = x.to(cuda).requires_grad_(True)
    wd = w.to(cuda).requires_grad_(True)
    out = GroupedGemmFunction.apply(xd, wd, cum, int((cum[1:] - cum[:-1]).max()), False)
    out.backward(dout.to(cuda))
    ref = _ref_fwd(x, w, cum)
    dx_ref = torch.zeros(rows, K); dw_ref = torch.zeros(G, N, K)
    for e in range(G):
        s, t = int(cum[e]), int(cum[e + 1])
        dx_ref[s:t] = dout[s:t].float() @ w[e].float()
        dw_ref[e] = dout[s:t].float().t() @ x[s:t].float()
    tag = (G, rows, N, K, kind)
    assert max_abs(out.float().cpu(), ref) <= 2e-2 * max(1.0, float(ref.abs().max())), tag
    assert_bf16_parity(out, ref, *ONE_ROUNDING, tag=f"ggemm_random{tag} fwd")
    assert_bf16_parity(xd.grad, dx_ref, *ONE_ROUNDING, tag=f"ggemm_random{tag} dgrad")
    assert max_abs(wd.grad.float().cpu(), dw_ref) <= 1e-2 * max(1.0, float(dw_ref.abs().max())), tag
    if float(dw_ref.abs().mean()) > 0:
        assert_bf16_parity(wd.grad, dw_ref, *ONE_ROUNDING, tag=f"ggemm_random{tag} wgrad")


@pytest.mark.parametrize("sizes", sorted(SWEEP_SIZES))
@pytest.mark.parametrize("seed", list(range(12)))
def test_gathered_merged_mlp_random_shapes(cuda, seed, sizes):
    """Seeded sweep of the bit-identity between the GEMMs that read tokens through input_indices and
    gather-then-GEMM, over token counts, top-k, expert windows and sizes."""
    from optimus.models.common.moe import (GatheredMergedMLPFunction, MergedMLPFunction,
                                           PrepareInputForGroupGemmFunction, build_token_permutation)
    from util import routed_experts
    rng = np.random.RandomState(99 + seed)
    N = int(rng.choice([4, 8, 16, 64]))
    K = int(rng.choice([1, 2, min(4, N)]))
    T = int(rng.choice([5, 64, 300, 1024, 5000]))
    H = int(rng.choice([128, 256, 384, 512] if sizes == "multiples_of_128" else [8, 72, 200, 328, 520]))
    I = int(rng.choice([128, 256, 384] if sizes == "multiples_of_128" else [8, 40, 136, 264]))
    start = int(rng.choice([0, N // 4]))
    end = int(rng.choice([N, max(start + 1, N - N // 4)]))
    G = end - start
    g = torch.Generator().manual_seed(seed)
    se = routed_experts(T, N, K, seed=seed, skew=float(rng.choice([0.0, 1.0]))).to(cuda)
    cum, cum_ep, ii, oi, _ = build_token_permutation(se, start, end)
    rows = int(cum[-1].item())
    ii, oi = ii[:rows], oi[:rows]
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ws = [(torch.randn(G, I, H, generator=g) * 0.05).to(torch.bfloat16),
          (torch.randn(G, I, H, generator=g) * 0.05).to(torch.bfloat16),
          (torch.randn(G, H, I, generator=g) * 0.05).to(torch.bfloat16)]
    dy = torch.randn(rows, H, generator=g).to(torch.bfloat16).to(cuda)
    results = []
    for gathered in (False, True):
        xd = x.to(cuda).requires_grad_(True)
        wd = [w.to(cuda).requires_grad_(True) for w in ws]
        if gathered:
            y = GatheredMergedMLPFunction.apply(xd, ii, cum_ep, oi, *wd, cum)
        else:
            y = MergedMLPFunction.apply(PrepareInputForGroupGemmFunction.apply(xd, ii, cum_ep, oi), *wd, cum)
        y.backward(dy)
        results.append([y.detach(), xd.grad] + [w.grad for w in wd])
    for name, a, b in zip(("y", "dx", "dw_gate", "dw_up", "dw_down"), *results):
        assert torch.equal(a, b), (name, T, K, N, start, end, I, H)


@pytest.mark.parametrize("G,rows,N,K", [(4096, 9000, 128, 256), (4097, 9000, 256, 128), (5000, 6000, 128, 128)])
def test_wgrad_with_thousands_of_experts(cuda, G, rows, N, K):
    """The weight gradient has no limit on the number of experts (the forward/dgrad tile table has).
    Up to 4096 experts its tiles are split over the XCDs by estimated work, above that by count:
    both sides of that threshold, most experts with 0-3 rows, against per-expert fp32 matmul."""
    from optimus import _native as n
    g = torch.Generator().manual_seed(G)
    c = torch.bincount(torch.randint(0, G, (rows,), generator=g), minlength=G)
    cum = torch.zeros(G + 1, dtype=torch.int32)
    cum[1:] = torch.cumsum(c, 0)
    dy = torch.randn(rows, N, generator=g).to(torch.bfloat16)
    x = torch.randn(rows, K, generator=g).to(torch.bfloat16)
    dyd, xd, cumd = dy.to(cuda), x.to(cuda), cum.to(cuda)
    dw = torch.full((G, N, K), float("nan"), dtype=torch.bfloat16, device=cuda)
    n.check(n.lib().om_grouped_gemm_wgrad(n.ptr(dyd), n.ptr(xd), n.ptr(dw), n.ptr(cumd), rows, G, N, K, 0,
                                          n.stream()), "om_grouped_gemm_wgrad")
    got = dw.float().cpu()
    assert bool(torch.isfinite(got).all())      # every tile of every expert was written
    ref = torch.zeros(G, N, K)
    for e in torch.nonzero(c).flatten().tolist():
        s, t = int(cum[e]), int(cum[e + 1])
        ref[e] = dy[s:t].float().t() @ x[s:t].float()
    assert max_abs(got, ref) <= 1e-2 * max(1.0, float(ref.abs().max()))
    assert float(got[c == 0].abs().max()) == 0.0


def test_operands_beyond_2_31_elements(cuda):
    """Activations of 1.1M rows x 2048 (2.25e9 elements, 4.5 GB): every product of the merged MLP,
    forward and backward, reads or writes a tensor past the 2^31-element mark.  Rows at the start,
    around the mark and at the end are checked against fp32 per-expert products, and so are the
    weight gradients of the expert whose rows straddle the mark and of the last one."""
    from optimus.models.common.moe import MergedMLPFunction
    rows, H, I, G = 1_100_000, 2048, 128, 4
    assert rows * H > (1 << 31)
    cum = torch.tensor([0, 500_000, 1_000_000, 1_099_000, rows], dtype=torch.int32)
    gen = torch.Generator(device=cuda).manual_seed(77)
    x = torch.randn(rows, H, device=cuda, dtype=torch.bfloat16, generator=gen).requires_grad_(True)
    dy = torch.randn(rows, H, device=cuda, dtype=torch.bfloat16, generator=gen)
    ws = [(torch.randn(shape, device=cuda, dtype=torch.float32, generator=gen) * 0.03).to(torch.bfloat16).requires_grad_(True)
          for shape in ((G, I, H), (G, I, H), (G, H, I))]
    y = MergedMLPFunction.apply(x, *ws, cum.to(cuda))
    y.backward(dy)
    torch.cuda.synchronize()
    mark = (1 << 31) // H
    picks = torch.cat([torch.arange(0, 48), torch.arange(mark - 40, mark + 40), torch.arange(999_980, 1_000_020),
                       torch.arange(rows - 48, rows)])
    expert_of = torch.bucketize(picks, cum[1:].long(), right=True)
    wf = [w.detach().float().cpu() for w in ws]
    for e in range(G):
        sel = picks[expert_of == e]
        if sel.numel() == 0:
            continue
        xr = x.detach()[sel.to(cuda)].float().cpu().requires_grad_(True)
        yr = (torch.nn.functional.silu(xr @ wf[0][e].t()) * (xr @ wf[1][e].t())) @ wf[2][e].t()
        yr.backward(dy[sel.to(cuda)].float().cpu())
        assert_bf16_parity(y.detach()[sel.to(cuda)], yr, *MLP_BARS["out"], tag=f"beyond2^31 expert {e} y")
        assert_bf16_parity(x.grad[sel.to(cuda)], xr.grad, *MLP_BARS["grad"], tag=f"beyond2^31 expert {e} dx")
    for e in (2, 3):       # rows 1,000,000..1,099,000 straddle the mark; 1,099,000.. lie beyond it
        s0, s1 = int(cum[e]), int(cum[e + 1])
        xr = x.detach()[s0:s1].float().cpu()
        p = [w[e].clone().requires_grad_(True) for w in wf]
        yr = (torch.nn.functional.silu(xr @ p[0].t()) * (xr @ p[1].t())) @ p[2].t()
        yr.backward(dy[s0:s1].float().cpu())
        for name, w, r in zip(("dwg", "dwu", "dwd"), ws, p):
            assert_bf16_parity(w.grad[e], r.grad, *MLP_BARS["grad"], tag=f"beyond2^31 expert {e} {name}")


@pytest.mark.parametrize("N,K", [(320, 192), (192, 2048), (1000, 328)])
def test_few_rows_kernels_give_the_bits_of_the_direct_load_kernels(cuda, N, K):
    """Experts with few rows run kernels that stage their operands through registers (the weights two
    contraction steps ahead); they are meant to change when data arrives in LDS, not what is summed.
    The same light experts are computed twice through the C ABI: alone (fewer than 256 rows per expert
    on average: the register-staged kernels), and followed by one heavy expert that lifts the average
    above 256 rows (the direct-load kernels; sizes that keep both launches on the 128x128 tile).  The
    light experts' rows must agree bit for bit, forward and input gradient."""
    from optimus import _native as n
    from util import bits
    g = torch.Generator().manual_seed(N + K)
    G = 12
    light = torch.randint(0, 90, (G,), generator=g)
    light[3] = 0
    rows_light = int(light.sum())
    heavy = (G + 1) * 256 + 64 - rows_light          # lifts the mean above 256 rows per expert
    cum_a = torch.zeros(G + 1, dtype=torch.int32); cum_a[1:] = torch.cumsum(light, 0)
    cum_b = torch.cat([cum_a, torch.tensor([rows_light + heavy], dtype=torch.int32)])
    rows_b = rows_light + heavy
    x = torch.randn(rows_b, K, generator=g).to(torch.bfloat16).to(cuda)
    dout = torch.randn(rows_b, N, generator=g).to(torch.bfloat16).to(cuda)
    w = (torch.randn(G + 1, N, K, generator=g) * 0.05).to(torch.bfloat16).to(cuda)
    P = n.ptr
    res = []
    for cum, rows, experts in ((cum_a, rows_light, G), (cum_b, rows_b, G + 1)):
        cum = cum.to(cuda)
        out = torch.zeros(rows_b, N, dtype=torch.bfloat16, device=cuda)
        dx = torch.zeros(rows_b, K, dtype=torch.bfloat16, device=cuda)
        n.check(n.lib().om_grouped_gemm_fwd(P(x), P(w), P(out), P(cum), rows, experts, N, K, 0, n.stream()), "fwd")
        n.check(n.lib().om_grouped_gemm_dgrad(P(dout), P(w), P(dx), P(cum), rows, experts, N, K, 0, n.stream()), "dgrad")
        torch.cuda.synchronize()
        res.append((out[:rows_light], dx[:rows_light]))
    assert rows_light < G * 256 and rows_b >= (G + 1) * 256
    assert float(res[0][0].float().abs().max()) > 0
    assert (bits(res[0][0]) == bits(res[1][0])).all()
    assert (bits(res[0][1]) == bits(res[1][1])).all()
