"""Helpers shared by the tests."""
import numpy as np
import torch


def bits(t):
    """torch tensor -> numpy; bf16 as raw uint16 bit patterns."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def from_bits(a, dtype):
    if dtype == torch.bfloat16:
        return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)
    return torch.from_numpy(np.ascontiguousarray(a))


def max_abs(a, b):
    return float((a.detach().double() - b.detach().double()).abs().max())


def mean_rel(a, b):
    """mean(|a-b|) / mean(|b|) — the layer-parity figure of merit."""
    a, b = a.detach().double(), b.detach().double()
    return float((a - b).abs().mean() / b.abs().mean().clamp_min(1e-30))


def routed_experts(T, N, K, seed, skew=0.0):
    """Distinct experts per token [T,K] int64, optionally Zipf-skewed."""
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, N, generator=g)
    if skew:
        rank = torch.randperm(N, generator=g) + 1
        logits = logits - skew * torch.log(rank.float())
    return torch.topk(logits, K, dim=1).indices


def bf16_floor(ref):
    """mean_rel of the ideally rounded reference: what a single bf16 rounding of `ref` costs
    (1.41e-3 for Gaussian data).  No kernel with a bf16 result can be closer to `ref` than this."""
    ref = ref.detach().float()
    return mean_rel(ref.to(torch.bfloat16).float(), ref)


_PARITY_LOG = []


def assert_bf16_parity(got, ref, excess, cap, tag="", max_abs_bar=None):
    """The bf16 parity bar as an EXCESS over an ideally rounded oracle:
        mean_rel(got, ref) <= excess * mean_rel(bf16(ref), ref)   and   mean_rel(got, ref) <= cap.
    `excess` says how many independent bf16 roundings' worth of error the chain of kernels behind
    `got` may add up to (a single product rounded once: just above 1; a whole layer, whose g, u, h
    and y are each rounded on the way as in the reference: 2-3); `cap` is an absolute ceiling near
    the measured figure, so that a lost accumulation or a dropped term cannot hide under the ratio
    when the reference itself is small.  Returns the measured mean_rel."""
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    m, floor = mean_rel(got, ref), bf16_floor(ref)
    _PARITY_LOG.append((tag, m, floor, m / max(floor, 1e-30), excess, cap))
    assert m <= excess * floor, (tag, "mean_rel", m, "floor", floor, "ratio", m / floor, "allowed", excess)
    assert m <= cap, (tag, "mean_rel", m, "cap", cap)
    if max_abs_bar is not None:
        ma = max_abs(got, ref)
        assert ma <= max_abs_bar, (tag, "max_abs", ma, max_abs_bar)
    return m


def dump_parity_log(path):
    with open(path, "a") as f:
        for tag, m, floor, ratio, excess, cap in _PARITY_LOG:
            f.write(f"{tag:60s} mean_rel {m:.3e} floor {floor:.3e} ratio {ratio:5.2f} (allowed {excess}, cap {cap:.1e})\n")
