"""Seeded synthetic inputs for the five benchmark / parity configurations of the hot path.

Everything is generated on the CPU with torch.Generator().manual_seed(seed) in fp32 and rounded to
the configuration's dtype, so a CPU checker and the GPU path see identical bits.
  C1 tiny MoE (fp32 reference case): T=2048 H=256  N=8   K=2 I=512,  renormalised top-2, seed 1001
  C2 AdamW 6.9e9 parameters                                                          seed 1002
  C3 OLMoE-1B-7B shape:            T=16384 H=2048 N=64  K=8 I=1024                   seed 1003
  C4 skewed small batch:           T=512   H=2048 N=64  K=8 I=1024, Zipf(1.2) bias   seed 1004
  C5 DeepSeek-V3 share:            T=8192  H=7168 N=256 (32 local) K=8 I=2048 + shared, seed 1005
"""
import math

import torch

MOE_SHAPES = {
    "C1": dict(T=2048, H=256, N=8, K=2, I=512, norm_topk_prob=True, seed=1001),
    "C3": dict(T=16384, H=2048, N=64, K=8, I=1024, norm_topk_prob=False, seed=1003),
    "C4": dict(T=512, H=2048, N=64, K=8, I=1024, norm_topk_prob=False, seed=1004),
}
DSV3_SHAPE = dict(T=8192, H=7168, N=256, NR=32, K=8, I=2048, n_group=8, topk_group=4,
                  routed_scaling_factor=2.5, norm_topk_prob=True, seed=1005)
ADAMW = dict(n=6_900_000_000, lr=4e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1, step_id=99,
             seed=1002)


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def moe_inputs(name, dtype=torch.bfloat16, scale_tokens=1.0):
    """-> dict(x [T,H], gate_w [N,H], w_gate/w_up [N,I,H], w_down [N,H,I], dout [T,H],
    router_logits_bias [N] or None, cfg).  `scale_tokens` < 1 shrinks T (for CPU checks)."""
    cfg = dict(MOE_SHAPES[name])
    T = max(8, int(cfg["T"] * scale_tokens) // 8 * 8)
    cfg["T"] = T
    H, N, I = cfg["H"], cfg["N"], cfg["I"]
    g = _gen(cfg["seed"])
    x = torch.randn(T, H, generator=g)
    gate_w = torch.randn(N, H, generator=g) * 0.02
    w_gate = torch.randn(N, I, H, generator=g) * 0.02
    w_up = torch.randn(N, I, H, generator=g) * 0.02
    w_down = torch.randn(N, H, I, generator=g) * 0.02
    dout = torch.randn(T, H, generator=g)
    out = dict(cfg=cfg, x=x.to(dtype), gate_w=gate_w.to(dtype), w_gate=w_gate.to(dtype),
               w_up=w_up.to(dtype), w_down=w_down.to(dtype), dout=dout.to(dtype), logits=None)
    if name == "C4":
        # router logits injected directly: N(0,1) + b_e, b_e = -1.2 ln(rank_e), rank = seeded
        # permutation of 1..N  (a Zipf(1.2) popularity over experts)
        rank = torch.randperm(N, generator=g) + 1
        bias = -1.2 * torch.log(rank.float())
        out["logits"] = torch.randn(T, N, generator=g) + bias
    return out


def dsv3_inputs(dtype=torch.bfloat16, scale_tokens=1.0, scale_hidden=1.0, seed=None):
    cfg = dict(DSV3_SHAPE)
    if seed is not None:
        cfg["seed"] = seed
    cfg["T"] = max(8, int(cfg["T"] * scale_tokens) // 8 * 8)
    cfg["H"] = max(128, int(cfg["H"] * scale_hidden) // 128 * 128)
    cfg["I"] = max(128, int(cfg["I"] * scale_hidden) // 128 * 128)
    T, H, N, NR, I = cfg["T"], cfg["H"], cfg["N"], cfg["NR"], cfg["I"]
    g = _gen(cfg["seed"])
    s = 0.006 / math.sqrt(scale_hidden)  # keeps the logit spread of the full-size case
    return dict(cfg=cfg,
                x=torch.randn(T, H, generator=g).to(dtype),
                router_w=(torch.randn(N, H, generator=g) * s),
                bias=torch.randn(N, generator=g) * 0.1,
                w_gate=(torch.randn(NR, I, H, generator=g) * s).to(dtype),
                w_up=(torch.randn(NR, I, H, generator=g) * s).to(dtype),
                w_down=(torch.randn(NR, H, I, generator=g) * s).to(dtype),
                ws_gate=(torch.randn(I, H, generator=g) * s).to(dtype),
                ws_up=(torch.randn(I, H, generator=g) * s).to(dtype),
                ws_down=(torch.randn(H, I, generator=g) * s).to(dtype),
                dout=torch.randn(T, H, generator=g).to(dtype))


def adamw_chunk(n, seed=ADAMW["seed"], chunk_id=0, device="cpu"):
    """One chunk of the C2 state: grad N(0,1e-3) bf16, master N(0,0.02), m N(0,1e-4),
    v |N(0,1e-6)|, param = bf16(master).  Generated on `device` with its own generator, so the
    GPU benchmark can fill 6.9e9 elements quickly; parity tests generate on the CPU and copy."""
    g = torch.Generator(device=device).manual_seed(seed + 7919 * chunk_id)
    grad = (torch.randn(n, generator=g, device=device) * 1e-3).to(torch.bfloat16)
    master = torch.randn(n, generator=g, device=device) * 0.02
    m = torch.randn(n, generator=g, device=device) * 1e-4
    v = (torch.randn(n, generator=g, device=device) * 1e-6).abs()
    return dict(grad=grad, master=master, exp_avg=m, exp_avg_sq=v, param=master.to(torch.bfloat16))
