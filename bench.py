#!/usr/bin/env python3
"""Benchmark of the MoE-layer + flat-buffer AdamW hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Primary workload (the `value`): one forward+backward of the OLMoE-1B-7B-shape MoE layer
(BASELINE config C3: 16384 tokens, hidden 2048, 64 experts, top-8, ffn 1024, bf16, fp32 router
logits), inputs resident in HBM; a step includes router, permutation, the nine expert GEMM
products (all weight gradients), combine and the router/gate backward.
Secondary workload (the `adamw` object of the same JSON line): the flat-buffer mixed-precision
AdamW step over 6.9e9 parameters (BASELINE config C2).

Kernel durations come from HIP events recorded on the launch stream around the C-ABI calls.  An
untimed profiling pass brackets every call (the `kernels` table, the all-GEMM aggregate, and which
entry point is dominant); inside the timed steps only the dominant entry point's launches are
bracketed, because every event pair leaves a gap of about 10 us on the stream, and the roofline
figure is taken from those.  The CPU baselines time the oracle's PyTorch-CPU restatements of the
reference path on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "optimus-lm_amd"))

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# HBM bytes per launch (read + write) come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# same command, scaled by what the counters read for a plain 1 GiB copy: counters cannot be collected
# inside the timed run, so the figures are kept in a data file next to the kernels, together with the
# command and the digest of the kernel source they were measured on.  A figure whose source has
# changed since is not reported (traffic: null).
MIB = float(1 << 20)
TRAFFIC_FILE = os.path.join(ROOT, "optimus-lm_amd", "csrc", "hbm_traffic_measured.json")


def source_digest(name):
    import hashlib
    with open(os.path.join(ROOT, "optimus-lm_amd", "csrc", name), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def measured_traffic_bytes(entry):
    """Measured HBM bytes per launch of a C-ABI entry point, or None when there is no figure for
    the kernel source as it is now."""
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    rec = table.get("entries", {}).get(entry)
    if rec is None or table.get("source_digest", {}).get(rec["source"]) != source_digest(rec["source"]):
        return None
    return (rec["fetch_mib"] + rec["write_mib"]) * MIB

GEMM_ENTRY_PRODUCTS = {     # C-ABI entry -> number of [rows x N x K] products per launch
    "om_merged_mlp_gate_up_fwd": 2, "om_grouped_gemm_fwd": 1, "om_grouped_gemm_wgrad": 1,
    "om_merged_mlp_gate_up_fwd_gathered": 2, "om_grouped_gemm_wgrad_gathered": 1,
    "om_merged_mlp_gate_up_fwd_weighted": 2, "om_grouped_gemm_wgrad_gathered_out": 1,
    "om_merged_mlp_down_dgrad_weighted": 1,
    "om_merged_mlp_down_dgrad": 1, "om_merged_mlp_gate_up_dgrad": 2, "om_grouped_gemm_dgrad": 1,
    "om_grouped_gemm_wgrad_accumulate": 1, "om_grouped_gemm_wgrad_gathered_accumulate": 1,
    "om_grouped_gemm_wgrad_gathered_out_accumulate": 1,
}


def build_block(inp, device):
    import torch
    from optimus.mapper import ParallelDpPpEpTpMapper
    from optimus.models.common.moe import FastOlmoeParallelSparseMoeBlock
    from optimus.models.olmoe.configuration_olmoe import OlmoeParallelConfig
    c = inp["cfg"]
    cfg = OlmoeParallelConfig(hidden_size=c["H"], intermediate_size=c["I"], num_experts=c["N"],
                              num_experts_per_tok=c["K"], norm_topk_prob=c["norm_topk_prob"],
                              use_fast_moe=True, use_merged_mlp_in_fast_moe=True)
    cfg.router_logits_fp32 = True
    blk = FastOlmoeParallelSparseMoeBlock(cfg, ParallelDpPpEpTpMapper()).to(device).to(torch.bfloat16)
    with torch.no_grad():
        blk.gate.weight.copy_(inp["gate_w"])
        blk.experts.gate_proj_merged_weight.copy_(inp["w_gate"])
        blk.experts.up_proj_merged_weight.copy_(inp["w_up"])
        blk.experts.down_proj_merged_weight.copy_(inp["w_down"])
    return blk


def bench_moe(args, device):
    import torch
    import synthetic_configs as sc
    from optimus import _native
    inp = sc.moe_inputs("C3")
    c = inp["cfg"]
    T, H, I, K = c["T"], c["H"], c["I"], c["K"]
    blk = build_block(inp, device)
    x = inp["x"].to(device).view(4, T // 4, H).requires_grad_(True)
    dout = inp["dout"].to(device).view(4, T // 4, H)

    def step():
        for p in blk.parameters():
            p.grad = None
        x.grad = None
        out, _ = blk(x)
        out.backward(dout)

    def run(n, only=None):
        """n steps with HIP events around the launches of the entry points in `only` (all if None);
        returns (ms per step, {entry: [durations in ms]})."""
        torch.cuda.synchronize()
        _native.launch_filter = only
        _native.launch_log = []
        t0 = time.perf_counter()
        for _ in range(n):
            step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        log, _native.launch_log = _native.launch_log, None
        _native.launch_filter = None
        per = {}
        for name, a, b in log:
            per.setdefault(name, []).append(a.elapsed_time(b))
        return (t1 - t0) * 1e3 / n, per

    for _ in range(args.warmup):
        step()
    # Profiling pass (not the metric): every entry point bracketed by events, which gives the per-kernel
    # table and names the dominant kernel.  An event pair costs a gap of about 10 us on the stream,
    # so the timed steps below bracket the dominant entry point only.
    _, per = run(max(3, min(args.steps, 10)))
    n_profiled = max(3, min(args.steps, 10))
    TR = T * K
    prod_flops = 2.0 * TR * H * I
    gemm_ms = sum(sum(v) for k, v in per.items() if k in GEMM_ENTRY_PRODUCTS) / n_profiled
    kernels = {k: {"launches_per_step": len(v) / n_profiled, "avg_ms": sum(v) / len(v)}
               for k, v in sorted(per.items())}
    # dominant kernel = the entry point with the largest summed duration; among entry points within 5 % of
    # it (one launch of two products against two launches of one product each sum to about the same), the
    # one with the longest launch, so that the choice does not flip from run to run
    summed = {k: sum(v) for k, v in per.items() if k in GEMM_ENTRY_PRODUCTS}
    dom = max((k for k in summed if summed[k] >= 0.95 * max(summed.values())), key=lambda k: summed[k] / len(per[k]))
    # The timed region: exactly args.steps steps, the dominant kernel's launches timed live.
    ms_per_step, per_dom = run(args.steps, only={dom})
    dom_avg_s = sum(per_dom[dom]) / len(per_dom[dom]) * 1e-3
    achieved = GEMM_ENTRY_PRODUCTS[dom] * prod_flops / dom_avg_s / 1e12
    roofline = {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 1),
                "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                "traffic": measured_traffic_bytes(dom),
                "all_expert_gemms": {"from": "untimed profiling pass with every entry point bracketed by events",
                                     "flops_per_step": 9 * prod_flops, "ms_per_step": round(gemm_ms, 3),
                                     "achieved": round(9 * prod_flops / (gemm_ms * 1e-3) / 1e12, 1),
                                     "frac": round(9 * prod_flops / (gemm_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)}}
    # The same step the way the reference's trainer runs it: the parameters' gradients are live views
    # of the optimizer's flat gradient buffer (optimizers.py:105-111) and every backward adds into
    # them (dist_train.py:154); the weight-gradient GEMMs do that sum in their epilogues.  Timed as
    # one micro-batch of an accumulation sequence, and with the buffer zeroed before every step.
    from optimus.optimizers import MixedPrecisionAdamW
    opt = MixedPrecisionAdamW(blk.parameters(), blk, lr=4e-4, dtype=torch.bfloat16, device=device,
                              skip_optimizer_step=True)

    def step_accumulating():
        x.grad = None
        out, _ = blk(x)
        out.backward(dout)

    def step_zeroed():
        opt.zero_grad()
        step_accumulating()

    def host_timed(fn, n):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / n
    opt.zero_grad()
    ms_acc = host_timed(step_accumulating, args.steps)
    ms_zero = host_timed(step_zeroed, args.steps)
    _native.launch_log = []
    step_zeroed()
    torch.cuda.synchronize()
    acc_log, _native.launch_log = _native.launch_log, None
    flat_grad_step = {
        "what": "the C3 step with every p.grad a live view of MixedPrecisionAdamW.flat_grad: weight gradients are "
                "added into the buffer by the GEMM epilogues (om_grouped_gemm_wgrad_*_accumulate)",
        "ms_per_step_accumulating": round(ms_acc, 3), "ms_per_step_with_zero_grad": round(ms_zero, 3),
        "over_detached_step": round(ms_acc / ms_per_step, 4),
        "wgrad_launches": sorted({nm for nm, _, _ in acc_log if "wgrad" in nm})}
    del opt
    # Yardstick, not part of the metric: the vendor library's dense bf16 GEMM (torch.matmul ->
    # hipBLASLt) on the two dense shapes with the same row count, contraction and data as the expert
    # products (one expert's weights for all 131072 rows).  With random operands the chip runs the
    # matrix cores power-limited, well below its nominal clock, so this is the practical ceiling the
    # grouped kernels can be held against on the same box.
    def dense_tflops(a, w):
        y = torch.empty(a.shape[0], w.shape[0], dtype=a.dtype, device=a.device)
        for _ in range(3):
            torch.matmul(a, w.t(), out=y)
        e0 = torch.cuda.Event(enable_timing=True); e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            torch.matmul(a, w.t(), out=y)
        e1.record(); torch.cuda.synchronize()
        return 2.0 * a.shape[0] * a.shape[1] * w.shape[0] / (e0.elapsed_time(e1) / 10 * 1e-3) / 1e12
    with torch.no_grad():
        a_h = x.detach().reshape(T, H).repeat(K, 1)                       # [TR, H]
        a_i = torch.randn(TR, I, device=device, dtype=torch.bfloat16)
        lib_up = dense_tflops(a_h, blk.experts.gate_proj_merged_weight[0])     # [TR,H] x [I,H]^T
        lib_down = dense_tflops(a_i, blk.experts.down_proj_merged_weight[0])   # [TR,I] x [H,I]^T
        del a_h, a_i
    roofline["library_dense_gemm_reference"] = {
        "what": "torch.matmul bf16 (vendor BLAS) on dense [131072,2048]x[2048,1024] and "
                "[131072,1024]x[1024,2048], same data distribution, same process",
        "tflops": [round(lib_up, 1), round(lib_down, 1)],
        "frac_of_peak": [round(lib_up / PEAK_BF16_TFLOPS, 4), round(lib_down / PEAK_BF16_TFLOPS, 4)]}
    del blk, x, dout
    torch.cuda.empty_cache()
    return dict(T=T, ms_per_step=ms_per_step, roofline=roofline, kernels=kernels, cfg=c,
                flat_grad_step=flat_grad_step)


def _timed_steps(step, warmup, steps):
    """(ms per step by the host clock, {entry point: summed ms over the steps}) for `steps` calls of
    step() with every C-ABI launch bracketed by HIP events."""
    import torch
    from optimus import _native
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    _native.launch_log = []
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    log, _native.launch_log = _native.launch_log, None
    per = {}
    for name, a, b in log:
        per[name] = per.get(name, 0.0) + a.elapsed_time(b)
    return ms, {k: v / steps for k, v in per.items()}


def _graph_replay_ms(step, steps):
    """ms per replay of step() recorded once into a HIP graph (torch.cuda.CUDAGraph): what the same
    kernels take without the host's per-launch work.  step() must allocate its gradients itself."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def bench_other_configs(args, device, with_cpu, only=None):
    """The other MoE configurations of BASELINE.json, each as whole-block forward+backward on the GPU:
    C1 (tiny, run in bf16 here; its float32 CPU reference path timed in full beside it), C4 (skewed
    small batch on injected router logits) and C5 (one rank's share of a DeepSeek-V3 layer).  For the
    two whose experts hold few rows (C4, the routed part of C5) the expert GEMMs are bound by
    streaming the expert weights, so both figures are given: MFMA fraction of the algorithmic flops
    and weight bytes per second (forward reads every local expert's three matrices once, the input
    gradients read them once more, the weight gradients write three matrices of the same size)."""
    import torch
    import synthetic_configs as sc
    from optimus.mapper import ParallelDpPpEpTpMapper
    from optimus.models.common.moe import (MergedMLPFunction, RoutedMLPFunction, SoftmaxTopkRouterFunction,
                                           expert_computation)
    steps = max(3, min(args.steps, 10))
    out = {}

    def gemm_ms(per):
        return sum(v for k, v in per.items() if k in GEMM_ENTRY_PRODUCTS)

    def entry(T, ms, per, flops, weight_bytes=None, extra=None, bound="mfma", traffic=None):
        g = gemm_ms(per)
        tflops = flops / (g * 1e-3) / 1e12
        e = {"ms_per_step": round(ms, 4), "tokens_per_s": round(T / (ms * 1e-3), 1),
             "expert_gemm_ms": round(g, 4), "expert_gemm_flops": flops,
             "mfma_frac": round(tflops / PEAK_BF16_TFLOPS, 4)}
        if weight_bytes is not None:
            e["weight_stream_gb_per_s"] = round(weight_bytes / (g * 1e-3) / 1e9, 1)
            e["weight_stream_hbm_frac"] = round(weight_bytes / (g * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
            e["weight_bytes_per_step"] = weight_bytes
        # the configuration's own roofline object, over all its expert-GEMM launches
        if bound == "hbm":
            gbs = weight_bytes / (g * 1e-3) / 1e9
            e["roofline"] = {"bound": "hbm", "kernel": "all expert GEMM launches of the step (weight streaming)",
                             "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": traffic}
        else:
            e["roofline"] = {"bound": "mfma", "kernel": "all expert GEMM launches of the step",
                             "achieved": round(tflops, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                             "frac": round(tflops / PEAK_BF16_TFLOPS, 4), "traffic": None}
        e["expert_gemm_launches_ms"] = {k: round(v, 4) for k, v in sorted(per.items()) if k in GEMM_ENTRY_PRODUCTS}
        if extra:
            e.update(extra)
        return e

    # ---- C1 -----------------------------------------------------------------------------------
    if only in (None, "C1"):
        inp = sc.moe_inputs("C1")
        c = inp["cfg"]
        blk = build_block(inp, device)
        x = inp["x"].to(device).view(1, c["T"], c["H"]).requires_grad_(True)
        dout = inp["dout"].to(device).view_as(x)

        def step_c1():
            for p in blk.parameters():
                p.grad = None
            x.grad = None
            o, _ = blk(x)
            o.backward(dout)
        ms, per = _timed_steps(step_c1, args.warmup, steps)
        flops = 18.0 * c["T"] * c["K"] * c["H"] * c["I"]
        graph_ms = _graph_replay_ms(step_c1, max(steps, 20))
        out["C1"] = entry(c["T"], ms, per, flops, extra={
            "graph_replay_ms_per_step": round(graph_ms, 4),
            "graph_replay_tokens_per_s": round(c["T"] / (graph_ms * 1e-3), 1),
            "workload": "C1 tiny MoE layer fwd+bwd (2048 tokens, hidden 256, 8 experts, top-2 renormalised, ffn 512), "
                        "bf16 on the GPU; about 25 launches, launch-bound when launched from Python "
                        "(ms_per_step); graph_replay_* is the same step recorded once into a HIP graph"})
        if with_cpu:
            from oracle import moe_layer as L
            cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
            torch.set_num_threads(cores)
            t = {k: inp[k].float().requires_grad_(True) for k in ("x", "gate_w", "w_gate", "w_up", "w_down")}
            best = None
            for _ in range(3):
                for v in t.values():
                    v.grad = None
                t0 = time.perf_counter()
                o, _ = L.olmoe_slow_block(t["x"], t["gate_w"], t["w_gate"], t["w_up"], t["w_down"], c["K"], True)
                o.backward(inp["dout"].float())
                dt = time.perf_counter() - t0
                best = dt if best is None else min(best, dt)
            out["C1"]["cpu_baseline"] = {"value": round(c["T"] / best, 1), "unit": "tokens/s", "cores": cores,
                                         "kind": "port", "sample": f"all 2048 tokens, float32, best of 3 ({best * 1e3:.1f} ms)"}
        del blk, x, dout

    # ---- C4 -----------------------------------------------------------------------------------
    if only in (None, "C4"):
        inp = sc.moe_inputs("C4")
        c = inp["cfg"]
        logits = inp["logits"].to(device)
        t = {k: inp[k].to(device).requires_grad_(True) for k in ("x", "w_gate", "w_up", "w_down")}
        dout = inp["dout"].to(device)
        routed = lambda hs, rw, ii, cum_ep, oi, si, cum, res: RoutedMLPFunction.apply(
            hs, rw, ii, cum_ep, oi, si, cum, res, True, t["w_gate"], t["w_up"], t["w_down"])
        fn = lambda gi, cum: MergedMLPFunction.apply(gi, t["w_gate"], t["w_up"], t["w_down"], cum)

        def step_c4():
            for v in t.values():
                v.grad = None
            w, e = SoftmaxTopkRouterFunction.apply(logits, c["K"], False, torch.bfloat16)
            o = expert_computation(t["x"], w.detach().requires_grad_(True), e, 0, c["N"], fn, c["N"],
                                   routed_experts_fn=routed)
            o.backward(dout)
        ms, per = _timed_steps(step_c4, args.warmup, steps)
        flops = 18.0 * c["T"] * c["K"] * c["H"] * c["I"]
        wbytes = 3 * 3 * c["N"] * c["H"] * c["I"] * 2
        with torch.no_grad():
            _, e = SoftmaxTopkRouterFunction.apply(logits, c["K"], False, torch.bfloat16)
            counts = torch.bincount(e.flatten(), minlength=c["N"])
        graph_ms = _graph_replay_ms(step_c4, max(steps, 20))
        one_pass = 3 * c["N"] * c["H"] * c["I"] * 2      # every expert's three matrices once
        per_launch = {   # weight bytes each entry point streams (reads, or writes for the weight gradients)
            "om_merged_mlp_gate_up_fwd_weighted": one_pass * 2 / 3, "om_grouped_gemm_fwd": one_pass / 3,
            "om_merged_mlp_down_dgrad_weighted": one_pass / 3, "om_merged_mlp_gate_up_dgrad": one_pass * 2 / 3,
            "om_grouped_gemm_wgrad_gathered": one_pass * 2 / 3, "om_grouped_gemm_wgrad_gathered_out": one_pass / 3}
        out["C4"] = entry(c["T"], ms, per, flops, wbytes, bound="hbm",
                          traffic=measured_traffic_bytes("C4:all_expert_gemm_launches"), extra={
            "weight_stream_gb_per_s_by_entry_point": {
                k: round(b / (per[k] * 1e-3) / 1e9, 1) for k, b in per_launch.items() if k in per},
            "graph_replay_ms_per_step": round(graph_ms, 4),
            "workload": "C4 OLMoE-shape layer under Zipf(1.2) routing, 512 tokens (router on injected logits, "
                        "permutation, expert GEMMs, combine; fwd+bwd)",
            "rows_per_expert": {"min": int(counts.min()), "median": int(counts.median()), "max": int(counts.max()),
                                "experts_with_at_most_8_rows": int((counts <= 8).sum())}})
        del t, logits, dout

    # ---- C5 -----------------------------------------------------------------------------------
    if only in (None, "C5"):
        from optimus.models.deepseek_v3.configuration_deepseek_v3 import DeepseekV3ParallelConfig
        from optimus.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3ParallelMoE
        inp = sc.dsv3_inputs()
        c = inp["cfg"]
        rank = 2
        c5cfg = DeepseekV3ParallelConfig(expert_parallelism=8)
        blk = DeepseekV3ParallelMoE(c5cfg, ParallelDpPpEpTpMapper(expert_parallelism=8, rank=rank)).to(device).to(torch.bfloat16)
        with torch.no_grad():
            blk.gate.weight.copy_(inp["router_w"]); blk.gate.e_score_correction_bias.copy_(inp["bias"])
            for i, m in enumerate(blk.experts):
                m.gate_proj.weight.copy_(inp["w_gate"][i]); m.up_proj.weight.copy_(inp["w_up"][i])
                m.down_proj.weight.copy_(inp["w_down"][i])
            blk.shared_experts.gate_proj.weight.copy_(inp["ws_gate"]); blk.shared_experts.up_proj.weight.copy_(inp["ws_up"])
            blk.shared_experts.down_proj.weight.copy_(inp["ws_down"])
        x = inp["x"].to(device).view(2, c["T"] // 2, c["H"]).requires_grad_(True)
        dout = inp["dout"].to(device).view_as(x)
        del inp

        def step_c5():
            for p in blk.parameters():
                p.grad = None
            x.grad = None
            o = blk(x)
            o.backward(dout)
        ms, per = _timed_steps(step_c5, max(2, args.warmup // 2), steps)
        # the same step with the routed-row count left on the device (nothing read back; the expert
        # activations are allocated for T*K rows): eager, and replayed from a HIP graph
        c5cfg.sync_free_expert_window = True
        ms_free, _ = _timed_steps(step_c5, 2, steps)
        graph_ms = _graph_replay_ms(step_c5, max(steps, 10))
        c5cfg.sync_free_expert_window = False
        with torch.no_grad():
            e, _ = blk.gate(x.detach())
            local = (e >= rank * c["NR"]) & (e < (rank + 1) * c["NR"])
            tr = int(local.sum())
            counts = torch.bincount((e[local] - rank * c["NR"]).flatten(), minlength=c["NR"])
        flops = 18.0 * (tr + c["T"]) * c["H"] * c["I"]
        wbytes = 3 * 3 * c["NR"] * c["H"] * c["I"] * 2
        out["C5"] = entry(c["T"], ms, per, flops, wbytes, extra={
            "workload": "C5 DeepSeek-V3-style layer, one GPU's share: 8192 tokens, hidden 7168, 32 local of 256 routed "
                        "experts (ffn 2048) + 1 shared expert, sigmoid group-limited top-8 router; fwd+bwd",
            "sync_free_window_ms_per_step": round(ms_free, 4), "graph_replay_ms_per_step": round(graph_ms, 4),
            "routed_rows_on_this_rank": tr,
            "rows_per_expert": {"min": int(counts.min()), "median": int(counts.median()), "max": int(counts.max())},
            "note": "expert_gemm_* and mfma_frac cover the routed and the shared expert's products together; "
                    "weight_stream_* counts the 32 routed experts' matrices only"})
        del blk, x, dout
        torch.cuda.empty_cache()
    return out


def bench_power_probe(args, device):
    """Not the metric: the five expert-GEMM entry points of the C3 step called directly on synthetic
    operands of the C3 shapes (uniformly random routing), once with N(0,1)-like data and once with
    all-zero activations and weights.  The arithmetic, the loads and the schedule are identical; only
    the switching activity in the matrix cores differs, so the ratio shows how far the chip's power
    limit, not the kernel's structure, sets the rate (pair it with `rocprofv3 --pmc GRBM_GUI_ACTIVE`
    for the engine clock)."""
    import torch
    from optimus import _native as n
    lib = n.lib()
    T, K, H, I, G = 16384, 8, 2048, 1024, 64
    TR = T * K
    g = torch.Generator(device=device).manual_seed(1)
    e = torch.topk(torch.randn(T, G, device=device, generator=g), K, dim=1).indices.flatten()
    input_indices = (torch.argsort(e, stable=True) // K).to(torch.int32).contiguous()
    cum = torch.zeros(G + 1, dtype=torch.int32, device=device)
    cum[1:] = torch.cumsum(torch.bincount(e, minlength=G), 0)
    bf = torch.bfloat16
    out = {}
    for kind in ("random", "zeros"):
        mk = (lambda *shape, scale=1.0: (torch.randn(*shape, device=device, generator=g) * scale).to(bf)) \
            if kind == "random" else (lambda *shape, scale=1.0: torch.zeros(*shape, device=device, dtype=bf))
        x, dfinal = mk(T, H), mk(T, H)
        wg, wu, wd = mk(G, I, H, scale=0.02), mk(G, I, H, scale=0.02), mk(G, H, I, scale=0.02)
        roww = torch.rand(TR, device=device, generator=g) if kind == "random" else torch.zeros(TR, device=device)
        gb, ub, hb = (torch.empty(TR, I, device=device, dtype=bf) for _ in range(3))
        dg, du = torch.empty_like(gb), torch.empty_like(gb)
        y, dx = torch.empty(TR, H, device=device, dtype=bf), torch.empty(TR, H, device=device, dtype=bf)
        dwg, dwu, dwd = torch.empty_like(wg), torch.empty_like(wu), torch.empty_like(wd)
        row_dot = torch.empty(I // 64, TR, device=device)
        P, st = n.ptr, n.stream()
        calls = [
            (2, lambda: lib.om_merged_mlp_gate_up_fwd_weighted(P(x), P(input_indices), T, P(wg), P(wu), P(roww), P(gb), P(ub), P(hb), P(cum), TR, G, I, H, 0, st)),
            (1, lambda: lib.om_grouped_gemm_fwd(P(hb), P(wd), P(y), P(cum), TR, G, H, I, 0, st)),
            (1, lambda: lib.om_merged_mlp_down_dgrad_weighted(P(dfinal), P(input_indices), T, P(wd), P(gb), P(ub), P(roww), P(dg), P(du), P(row_dot), P(cum), TR, G, I, H, 0, st)),
            (2, lambda: lib.om_merged_mlp_gate_up_dgrad(P(dg), P(du), P(wg), P(wu), P(dx), P(cum), TR, G, I, H, 0, st)),
            (1, lambda: lib.om_grouped_gemm_wgrad_gathered(P(dg), P(x), P(input_indices), T, P(dwg), P(cum), TR, G, I, H, 0, st)),
            (1, lambda: lib.om_grouped_gemm_wgrad_gathered(P(du), P(x), P(input_indices), T, P(dwu), P(cum), TR, G, I, H, 0, st)),
            (1, lambda: lib.om_grouped_gemm_wgrad_gathered_out(P(dfinal), P(input_indices), T, P(hb), P(dwd), P(cum), TR, G, H, I, 0, st)),
        ]

        def step():
            for _, fn in calls:
                n.check(fn(), "power probe")
        for _ in range(max(3, args.warmup)):
            step()
        torch.cuda.synchronize()
        a = torch.cuda.Event(enable_timing=True); b = torch.cuda.Event(enable_timing=True)
        reps = max(5, args.steps)
        a.record()
        for _ in range(reps):
            step()
        b.record(); torch.cuda.synchronize()
        ms = a.elapsed_time(b) / reps
        out[kind] = {"ms_per_nine_products": round(ms, 3),
                     "tflops": round(9 * 2.0 * TR * H * I / (ms * 1e-3) / 1e12, 1),
                     "frac_of_peak": round(9 * 2.0 * TR * H * I / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)}
        del x, dfinal, wg, wu, wd, gb, ub, hb, dg, du, y, dx, dwg, dwu, dwd
        torch.cuda.empty_cache()
    out["zeros_over_random"] = round(out["zeros"]["tflops"] / out["random"]["tflops"], 3)
    return out


def cpu_baseline_moe():
    """oracle.moe_layer.olmoe_slow_block (the reference's per-expert loop, fp32) forward+backward on
    1/16 of the C3 tokens with the full expert weights; tokens/s of that run."""
    import torch
    import synthetic_configs as sc
    from oracle import moe_layer as L
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    inp = sc.moe_inputs("C3", scale_tokens=1.0 / 16)
    c = inp["cfg"]
    t = {k: inp[k].float().requires_grad_(True) for k in ("x", "gate_w", "w_gate", "w_up", "w_down")}
    d = inp["dout"].float()
    t0 = time.perf_counter()
    out, _ = L.olmoe_slow_block(t["x"], t["gate_w"], t["w_gate"], t["w_up"], t["w_down"], c["K"],
                                c["norm_topk_prob"])
    out.backward(d)
    dt = time.perf_counter() - t0
    return {"value": round(c["T"] / dt, 1), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{c['T']} of 16384 tokens (1/16), all 64 experts' weights, fp32 PyTorch-CPU "
                      f"restatement of OlmoeParallelSparseMoeBlock fwd+bwd, {dt:.1f} s"}


def bench_adamw(args, device):
    import torch
    import synthetic_configs as sc
    from optimus import _native
    from optimus.optimizers import adamw_step_
    hp = sc.ADAMW
    n = hp["n"]
    free, _ = torch.cuda.mem_get_info()
    need = 16 * n * 1.05
    if free < need:
        return {"skipped": f"needs {need / 1e9:.0f} GB free HBM, have {free / 1e9:.0f} GB"}
    chunk = 1 << 26
    seedst = sc.adamw_chunk(chunk, device=device)
    reps = -(-n // chunk)
    st = {k: v.repeat(reps)[:n].contiguous() for k, v in seedst.items()}
    del seedst
    steps = max(3, min(args.steps, 10))

    def step(i):
        adamw_step_(st["param"], st["grad"], st["master"], st["exp_avg"], st["exp_avg_sq"],
                    hp["step_id"] + 1 + i, hp["lr"], hp["betas"][0], hp["betas"][1], hp["eps"],
                    hp["weight_decay"])

    # the memory clocks take a few seconds of load to reach their steady state after the idle
    # period of the CPU baseline: warm up untimed for about three seconds
    t_warm = time.perf_counter()
    i = 0
    while i < args.warmup or time.perf_counter() - t_warm < 3.0:
        step(i % 30)
        i += 1
        if i % 10 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    _native.launch_log = []
    t0 = time.perf_counter()
    for i in range(steps):
        step(40 + i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    log, _native.launch_log = _native.launch_log, None
    kern_ms = [a.elapsed_time(b) for _, a, b in log]
    avg_s = sum(kern_ms) / len(kern_ms) * 1e-3
    gbs = 28.0 * n / avg_s / 1e9

    # The gradient-norm pass and the update with the clip folded in (optimizers.py:136-160 then
    # :162-205): one plan over 54 equal "parameters", coefficient 1.0 so the data stay put.
    from optimus.optimizers import GradNormPlan
    n_par = 54
    sizes = [n // n_par] * (n_par - 1) + [n - (n // n_par) * (n_par - 1)]
    starts = [sum(sizes[:i]) for i in range(n_par)]
    plan = GradNormPlan(starts, sizes, device)
    one = torch.ones(1, dtype=torch.float32, device=device)

    def timed(fn, names, reps=5):
        fn(); fn()
        torch.cuda.synchronize()
        _native.launch_log = []
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        lg, _native.launch_log = _native.launch_log, None
        return sum(a.elapsed_time(b) for nm, a, b in lg if nm in names) / reps * 1e-3

    t_norm = timed(lambda: plan.run(st["grad"]), ("om_grad_sumsq", "om_grad_norm_clip_coef"))
    t_clip = {}
    for store in (True, False):
        t_clip[store] = timed(lambda: adamw_step_(
            st["param"], st["grad"], st["master"], st["exp_avg"], st["exp_avg_sq"], hp["step_id"] + 1,
            hp["lr"], hp["betas"][0], hp["betas"][1], hp["eps"], hp["weight_decay"], grad_scale=one,
            store_scaled_grad=store), ("om_adamw_step_clipped",))
    # What the update's access pattern reaches on this GPU with the arithmetic taken out: the same
    # 64-thread blocks, the same 14 B read + 14 B written per parameter, the same cache hints.
    t_probe = timed(lambda: _native.check(_native.lib().om_adamw_traffic_probe(
        _native.ptr(st["param"]), _native.ptr(st["grad"]), _native.ptr(st["master"]), _native.ptr(st["exp_avg"]),
        _native.ptr(st["exp_avg_sq"]), n, _native.stream()), "om_adamw_traffic_probe"), ("om_adamw_traffic_probe",))
    probe_gbs = 28.0 * n / t_probe / 1e9
    grad_clip = {
        "grad_norm_ms": round(t_norm * 1e3, 3), "grad_norm_gb_per_s": round(2.0 * n / t_norm / 1e9, 1),
        "clipped_step_ms": round(t_clip[True] * 1e3, 3),
        "clipped_step_gb_per_s": round(30.0 * n / t_clip[True] / 1e9, 1),
        "clipped_step_no_store_ms": round(t_clip[False] * 1e3, 3),
        "clipped_step_no_store_gb_per_s": round(28.0 * n / t_clip[False] / 1e9, 1),
        "note": "norm pass reads 2 B/param; clipped step = 28 B/param + 2 B/param when the scaled "
                "gradient is stored back; 54 parameter slices, 65536-element chunks"}
    # One rank's share of the same buffers under 8-way sharding (ShardedMixedPrecisionAdamW.step,
    # reference optimizers.py:398-479, without the collectives): norm of the shard, clip decision on
    # the device, update with the clip folded in and the clipped gradient stored back.
    shard = -(-n // (8 * 512)) * 512
    sh = {k: v[:shard] for k, v in st.items()}
    shard_plan = GradNormPlan([0], [shard], device)
    clip_buf = torch.zeros(2, dtype=torch.float32, device=device)

    def shard_step():
        norm = shard_plan.run(sh["grad"])[0]
        _native.check(_native.lib().om_shard_clip_multiplier(
            _native.ptr(norm), 0, _native.OM_BF16, 1.0, _native.ptr(clip_buf), _native.ptr(clip_buf) + 4,
            _native.stream()), "om_shard_clip_multiplier")
        adamw_step_(sh["param"], sh["grad"], sh["master"], sh["exp_avg"], sh["exp_avg_sq"], hp["step_id"] + 1,
                    hp["lr"], hp["betas"][0], hp["betas"][1], hp["eps"], hp["weight_decay"],
                    grad_scale=clip_buf[1:2], store_scaled_grad=True)
    t_shard = timed(shard_step, ("om_grad_sumsq", "om_grad_norm_clip_coef", "om_shard_clip_multiplier",
                                 "om_adamw_step_clipped"))
    sharded = {"what": "one rank's shard of C2 under 8-way sharding: shard norm, device-side clip decision, "
                       "clipped update storing the scaled gradient (4 launches, 32 B/param)",
               "shard_params": shard, "ms": round(t_shard * 1e3, 3),
               "gb_per_s": round(32.0 * shard / t_shard / 1e9, 1),
               "frac_of_peak": round(32.0 * shard / t_shard / 1e9 / PEAK_HBM_GBS, 4)}
    del st, sh, plan, shard_plan
    torch.cuda.empty_cache()
    return {"metric": "adamw_step_hbm_gb_per_s", "value": round(gbs, 1), "unit": "GB/s",
            "ms_per_step": round((t1 - t0) * 1e3 / steps, 3), "steps": steps, "dtype": "f32",
            "config": {"workload": "C2 flat-buffer mixed-precision AdamW, 6.9e9 params, bf16 "
                                   "param/grad + fp32 master/m/v, step 100"},
            "roofline": {"bound": "hbm", "kernel": "om_adamw_step", "achieved": round(gbs, 1),
                         "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4),
                         "traffic": measured_traffic_bytes("om_adamw_step"), "bytes_per_param": 28, "kernel_avg_ms": round(avg_s * 1e3, 3),
                         "streaming_ceiling": {
                             "what": "om_adamw_traffic_probe: the update kernel's loads and stores (14 B read + "
                                     "14 B written per parameter, same block shape and cache hints) without "
                                     "the arithmetic, same buffers, same process",
                             "gb_per_s": round(probe_gbs, 1), "frac_of_peak": round(probe_gbs / PEAK_HBM_GBS, 4),
                             "update_over_probe": round(gbs / probe_gbs, 4)}},
            "grad_clip": grad_clip, "sharded_step": sharded}


def cpu_baseline_adamw():
    """The reference's chunked 13-op torch sequence (oracle.adamw.adamw_step_torch) on 2^25 elements."""
    import torch
    import synthetic_configs as sc
    from oracle.adamw import adamw_step_torch
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    n = 1 << 25
    st = sc.adamw_chunk(n)
    hp = sc.ADAMW
    adamw_step_torch(st["param"], st["grad"], st["master"], st["exp_avg"], st["exp_avg_sq"], 98,
                     hp["lr"], hp["betas"], hp["eps"], hp["weight_decay"])
    reps = 3
    t0 = time.perf_counter()
    for i in range(reps):
        adamw_step_torch(st["param"], st["grad"], st["master"], st["exp_avg"], st["exp_avg_sq"],
                         99 + i, hp["lr"], hp["betas"], hp["eps"], hp["weight_decay"])
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(28.0 * n / dt / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"2^25 elements ({16 * n / 1e9:.2f} GB of state), the reference's 13 torch "
                      f"elementwise ops per chunk on CPU, {dt * 1e3:.0f} ms per step; GB/s on the "
                      "28 B/param algorithmic figure"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-cpu", action="store_true", help="leave out the CPU baselines")
    ap.add_argument("--skip-adamw", action="store_true", help="leave out the AdamW workload")
    ap.add_argument("--skip-other", action="store_true", help="leave out the C1 / C4 / C5 configurations")
    ap.add_argument("--only-config", choices=("C1", "C4", "C5"),
                    help="only run this one of the other configurations (for profiling)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="only run four 1 GiB device copies (calibrates the HBM traffic counters)")
    ap.add_argument("--power-probe", action="store_true",
                    help="only run the expert GEMMs on random and on all-zero operands (power-limit evidence)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU's hot path; --gpus must be 1 "
              "(no collectives or sharding are part of it)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from optimus import _native
    _native.lib()
    device = torch.device("cuda:0")
    if args.power_probe:
        print(json.dumps({"power_probe": bench_power_probe(args, device), "n_gpus": 1,
                          "note": "expert GEMM entry points on random vs all-zero operands; not the metric"}))
        return
    if args.copy_probe:
        # a device-to-device copy of known size: what FETCH_SIZE / WRITE_SIZE read for it gives the
        # factors that turn those counters into bytes
        n = 1 << 30
        src = torch.empty(n, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_probe": {"bytes_per_copy": n, "copies": 4}, "n_gpus": 1}))
        return
    if args.only_config:
        print(json.dumps({"other_configs": bench_other_configs(args, device, False, only=args.only_config),
                          "n_gpus": 1, "note": "one of the parity-test configurations; not the metric"}))
        return
    moe = bench_moe(args, device)
    out = {
        "metric": "olmoe_moe_layer_fwd_bwd_tokens_per_s", "value": round(moe["T"] / (moe["ms_per_step"] * 1e-3), 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(moe["ms_per_step"], 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "C3 OLMoE-1B-7B-shape MoE layer fwd+bwd: 16384 tokens (4x4096), hidden "
                               "2048, 64 experts, top-8, ffn 1024, fp32 router logits, no dropping"},
        "roofline": moe["roofline"], "kernels": moe["kernels"], "flat_grad_step": moe["flat_grad_step"],
    }
    # GPU workloads first, back to back: the seconds of CPU baseline in between would let the GPU
    # fall into its idle power state right before the HBM-bound measurement
    if not args.skip_other:
        out["other_configs"] = bench_other_configs(args, device, not args.skip_cpu)
    ad = None if args.skip_adamw else bench_adamw(args, device)
    if not args.skip_cpu:
        out["cpu_baseline"] = cpu_baseline_moe()
    if ad is not None:
        if not args.skip_cpu and "skipped" not in ad:
            ad["cpu_baseline"] = cpu_baseline_adamw()
        out["adamw"] = ad
    print(json.dumps(out))


if __name__ == "__main__":
    main()
    sys.stdout.flush()
