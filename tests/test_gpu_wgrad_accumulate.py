"""Weight gradients accumulated into a live gradient buffer inside the GEMM epilogue.

In the reference every p.grad is a view of the optimizer's flat gradient buffer
(optimus/optimizers.py:105-111) that is zeroed in place (:117-118) and accumulated into over the
micro-batches of a step (dist_train.py:154), so autograd ends each weight-gradient GEMM with an
in-place `p.grad += dW`.  The *_accumulate entry points do that sum in the epilogue.  The bar is
bit equality with the two-step form: the same GEMM writing a fresh dW, then torch's in-place add.
"""
import pytest
import torch

from util import bits
from test_gpu_ggemm import _counts

pytestmark = pytest.mark.gpu


def _call(name, *args):
    from optimus import _native as n
    n.check(getattr(n.lib(), name)(*args, n.stream()), name)


# (kind, G, rows, N, K): both tile shapes (256x256 needs N, K multiples of 256 and enough tiles),
# odd row counts (single trailing contraction step), experts without rows
ABI_CASES = [("ragged", 64, 4096, 256, 512), ("empties", 16, 777, 128, 256), ("uniform", 8, 1000, 512, 256),
             ("onehot", 9, 3000, 512, 256), ("ragged", 3, 5, 128, 128), ("ragged", 150, 6000, 128, 128),
             ("ragged", 8, 1000, 192, 320)]   # partial last tiles along both extents of dW


@pytest.mark.parametrize("kind,G,rows,N,K", ABI_CASES)
@pytest.mark.parametrize("form", ["plain", "gathered", "gathered_out"])
def test_accumulate_entry_points_equal_gemm_then_add(cuda, form, kind, G, rows, N, K):
    from optimus import _native as n
    g = torch.Generator().manual_seed(rows + N)
    T = max(rows // 2, 8)
    idx = torch.randint(0, T, (rows,), generator=g, dtype=torch.int32).to(cuda)
    dout_rows = T if form == "gathered_out" else rows
    in_rows = T if form == "gathered" else rows
    dout = torch.randn(dout_rows, N, generator=g).to(torch.bfloat16).to(cuda)
    x = torch.randn(in_rows, K, generator=g).to(torch.bfloat16).to(cuda)
    cum = _counts(kind, G, rows).to(cuda)
    pitch = N * K + 64                       # per-expert matrices at a constant pitch inside one buffer
    old = torch.randn(G * pitch, generator=g).to(torch.bfloat16).to(cuda)
    P = n.ptr

    def run(suffix, out):
        if form == "plain":
            _call("om_grouped_gemm_wgrad" + suffix, P(dout), P(x), P(out), P(cum), rows, G, N, K, pitch)
        elif form == "gathered":
            _call("om_grouped_gemm_wgrad_gathered" + suffix, P(dout), P(x), P(idx), T, P(out), P(cum), rows, G,
                  N, K, pitch)
        else:
            _call("om_grouped_gemm_wgrad_gathered_out" + suffix, P(dout), P(idx), T, P(x), P(out), P(cum), rows,
                  G, N, K, pitch)

    fresh = torch.zeros_like(old)
    run("", fresh)
    acc = old.clone()
    run("_accumulate", acc)
    view = lambda t: torch.as_strided(t, (G, N, K), (pitch, K, 1))
    expect = old.clone()
    view(expect).add_(view(fresh))           # torch's in-place bf16 add: fp32 sum, one rounding
    torch.cuda.synchronize()
    assert (bits(acc) == bits(expect)).all()
    # the padding between the experts' matrices is not touched
    gap = torch.as_strided(acc, (G, 64), (pitch, 1), N * K)
    assert (bits(gap) == bits(torch.as_strided(old, (G, 64), (pitch, 1), N * K))).all()
    # a second accumulation on top of the first
    run("_accumulate", acc)
    view(expect).add_(view(fresh))
    torch.cuda.synchronize()
    assert (bits(acc) == bits(expect)).all()


def test_accumulate_f32(cuda):
    from optimus import _native as n
    g = torch.Generator().manual_seed(5)
    G, rows, N, K = 6, 700, 128, 64
    dout = torch.randn(rows, N, generator=g).to(cuda)
    x = torch.randn(rows, K, generator=g).to(cuda)
    cum = _counts("empties", G, rows).to(cuda)
    old = torch.randn(G, N, K, generator=g).to(cuda)
    fresh = torch.empty_like(old)
    P = n.ptr
    _call("om_grouped_gemm_wgrad_f32", P(dout), P(x), P(fresh), P(cum), rows, G, N, K, 0)
    acc = old.clone()
    _call("om_grouped_gemm_wgrad_f32_accumulate", P(dout), P(x), P(acc), P(cum), rows, G, N, K, 0)
    torch.cuda.synchronize()
    assert torch.equal(acc, old + fresh)


def _olmoe_block(cuda, merged, fast=True, dtype=torch.bfloat16, seed=3):
    from optimus.mapper import ParallelDpPpEpTpMapper
    from optimus.models.common.moe import FastOlmoeParallelSparseMoeBlock
    from optimus.models.olmoe.configuration_olmoe import OlmoeParallelConfig
    from optimus.models.olmoe.modeling_olmoe import OlmoeParallelSparseMoeBlock
    cfg = OlmoeParallelConfig(hidden_size=256, intermediate_size=256, num_experts=8, num_experts_per_tok=2,
                              norm_topk_prob=True, use_fast_moe=True, use_merged_mlp_in_fast_moe=merged)
    cfg.router_logits_fp32 = True
    torch.manual_seed(seed)
    cls = FastOlmoeParallelSparseMoeBlock if fast else OlmoeParallelSparseMoeBlock
    blk = cls(cfg, ParallelDpPpEpTpMapper())
    for p in blk.parameters():
        torch.nn.init.normal_(p, std=0.05)
    return blk.to(cuda).to(dtype)


def _dsv3_block(cuda, seed=4):
    from optimus.mapper import ParallelDpPpEpTpMapper
    from optimus.models.deepseek_v3.configuration_deepseek_v3 import DeepseekV3ParallelConfig
    from optimus.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3ParallelMoE
    cfg = DeepseekV3ParallelConfig(hidden_size=256, moe_intermediate_size=128, n_routed_experts=16,
                                   num_experts_per_tok=4, n_group=4, topk_group=2, expert_parallelism=2)
    torch.manual_seed(seed)
    blk = DeepseekV3ParallelMoE(cfg, ParallelDpPpEpTpMapper(expert_parallelism=2, rank=1))
    for p in blk.parameters():
        torch.nn.init.normal_(p, std=0.05)
    return blk.to(cuda).to(torch.bfloat16)


def _two_backwards(blk, cuda, dtype, in_place):
    """flat_grad after two backward passes without zero_grad under MixedPrecisionAdamW, and the
    names of the C-ABI entry points the second pass launched."""
    from optimus import _native
    from optimus.models.common import moe
    from optimus.optimizers import MixedPrecisionAdamW
    opt = MixedPrecisionAdamW(blk.parameters(), blk, lr=1e-3, dtype=dtype, device=cuda)
    g = torch.Generator().manual_seed(11)
    xs = [torch.randn(2, 192, 256, generator=g).to(dtype).to(cuda) for _ in range(2)]
    ds = [torch.randn(2, 192, 256, generator=g).to(dtype).to(cuda) for _ in range(2)]
    moe.accumulate_weight_grads_in_place = in_place
    try:
        opt.zero_grad()
        names = []
        for i, (x, d) in enumerate(zip(xs, ds)):
            if i == 1:
                _native.launch_log = []
            out = blk(x)
            out = out[0] if isinstance(out, tuple) else out
            out.backward(d)
        torch.cuda.synchronize()
        names = [nm for nm, _, _ in _native.launch_log]
    finally:
        _native.launch_log = None
        moe.accumulate_weight_grads_in_place = True
    for p in blk.parameters():          # every gradient still is its view of the flat buffer
        assert p.grad.untyped_storage().data_ptr() == opt.flat_grad.untyped_storage().data_ptr()
    return opt.flat_grad.clone(), names


BLOCKS = {
    "fast_merged": lambda cuda: (_olmoe_block(cuda, True), torch.bfloat16),
    "fast_per_expert": lambda cuda: (_olmoe_block(cuda, False), torch.bfloat16),
    "slow_per_expert": lambda cuda: (_olmoe_block(cuda, False, fast=False), torch.bfloat16),
    "fast_merged_f32": lambda cuda: (_olmoe_block(cuda, True, dtype=torch.float32), torch.float32),
    "dsv3_window_and_shared": lambda cuda: (_dsv3_block(cuda), torch.bfloat16),
}


@pytest.mark.parametrize("which", sorted(BLOCKS))
def test_block_under_flat_buffer_optimizer_accumulates_in_the_epilogue(cuda, which):
    """Two backward passes without zero_grad: the flat gradient buffer is bit-identical whether the
    weight-gradient GEMMs add into it themselves or autograd adds their fresh results, and in the
    first form no plain weight-gradient launch (hence no separate accumulation pass) is left."""
    blk_a, dtype = BLOCKS[which](cuda)
    blk_b, _ = BLOCKS[which](cuda)
    fused, names_fused = _two_backwards(blk_a, cuda, dtype, True)
    plain, names_plain = _two_backwards(blk_b, cuda, dtype, False)
    assert (bits(fused) == bits(plain)).all()
    assert float(fused.float().abs().max()) > 0
    wgrads = [nm for nm in names_fused if nm.startswith("om_grouped_gemm_wgrad")]
    assert wgrads and all(nm.endswith("_accumulate") for nm in wgrads), wgrads
    assert not any(nm.endswith("_accumulate") for nm in names_plain)


def test_fresh_gradients_without_a_live_buffer(cuda):
    """Without an optimizer that owns the gradients (p.grad is None, or a tensor of its own) the
    functions return fresh gradients and autograd accumulates as usual."""
    from optimus import _native
    blk = _olmoe_block(cuda, True)
    x = torch.randn(1, 128, 256).to(torch.bfloat16).to(cuda)
    _native.launch_log = []
    try:
        for _ in range(2):
            blk(x)[0].backward(torch.ones_like(x))
        torch.cuda.synchronize()
        names = [nm for nm, _, _ in _native.launch_log]
    finally:
        _native.launch_log = None
    assert not any(nm.endswith("_accumulate") for nm in names)
    assert all(p.grad is not None for p in blk.parameters())


def test_accumulation_under_activation_checkpointing(cuda):
    """With the block's expert computation under torch's activation checkpoint (the reference's
    use_activation_checkpointing bit 0, moe.py:430-432, :612-616) the recomputed forward's backward
    still adds into the live gradient buffer, with the same bits as without checkpointing."""
    from optimus.optimizers import MixedPrecisionAdamW
    res = []
    for ckpt in (False, True):
        blk = _olmoe_block(cuda, True)
        blk.use_activation_checkpointing_for_moe = ckpt
        opt = MixedPrecisionAdamW(blk.parameters(), blk, lr=1e-3, dtype=torch.bfloat16, device=cuda)
        g = torch.Generator().manual_seed(21)
        opt.zero_grad()
        for _ in range(2):
            x = torch.randn(2, 128, 256, generator=g).to(torch.bfloat16).to(cuda).requires_grad_(True)
            blk(x)[0].backward(torch.randn(2, 128, 256, generator=g).to(torch.bfloat16).to(cuda))
        torch.cuda.synchronize()
        res.append(opt.flat_grad.clone())
    assert (bits(res[0]) == bits(res[1])).all() and float(res[0].float().abs().max()) > 0
