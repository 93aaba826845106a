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
