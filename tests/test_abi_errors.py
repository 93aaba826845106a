"""Error convention of the C ABI: every entry point validates its arguments before it touches the
HIP runtime and answers with a negative OM_ERR_* code — it never throws and never launches on bad
input.  These calls return from the validation, so they run without a GPU; the pointers are made-up
addresses that are never dereferenced on the host."""
import pytest

from optimus import _native as n

OK, NULL, DTYPE, SHAPE, ALIGN, LAUNCH, WORKSPACE = 0, -1, -2, -3, -4, -5, -6
P = 0x7f0000001000        # a 16-byte aligned, never dereferenced "device pointer"
ODD = P + 8               # misaligned
BF16, F32, I64 = n.OM_BF16, n.OM_F32, 1


@pytest.fixture(scope="module")
def lib():
    return n.lib()


def test_strerror_names_every_code(lib):
    texts = {c: lib.om_strerror(c).decode() for c in (OK, NULL, DTYPE, SHAPE, ALIGN, LAUNCH, WORKSPACE)}
    assert len(set(texts.values())) == 7 and all(texts.values())
    assert "unknown" in lib.om_strerror(-99).decode()


def test_adamw(lib):
    hp = (4e-4, 0.9, 0.95, 1e-8, 0.1)
    assert lib.om_adamw_step(P, P, P, P, P, 16, *hp, 1, 7, None) == DTYPE
    assert lib.om_adamw_step(P, P, P, P, P, 16, *hp, 0, BF16, None) == SHAPE      # step is 1-based
    assert lib.om_adamw_step(P, P, P, P, P, -1, *hp, 1, BF16, None) == SHAPE
    assert lib.om_adamw_step(P, P, P, P, P, 0, *hp, 1, BF16, None) == OK          # nothing to do
    assert lib.om_adamw_step(P, None, P, P, P, 16, *hp, 1, BF16, None) == NULL
    assert lib.om_adamw_step(None, P, P, P, P, 16, *hp, 1, BF16, None) == NULL    # bf16 mode needs param
    assert lib.om_adamw_step(P, P, ODD, P, P, 16, *hp, 1, BF16, None) == ALIGN
    assert lib.om_adamw_step_clipped(P, P, P, P, P, 16, *hp, 1, BF16, None, 1, None) == NULL   # no scale
    assert lib.om_adamw_step_clipped(P, P, P, P, P, 16, *hp, 1, 9, P, 1, None) == DTYPE


def test_grad_norm(lib):
    assert lib.om_grad_sumsq(P, 5, P, 4, P, None) == DTYPE
    assert lib.om_grad_sumsq(P, BF16, P, -1, P, None) == SHAPE
    assert lib.om_grad_sumsq(P, BF16, P, 0, P, None) == OK
    assert lib.om_grad_sumsq(None, BF16, P, 4, P, None) == NULL
    assert lib.om_grad_sumsq(ODD, BF16, P, 4, P, None) == ALIGN
    assert lib.om_grad_norm_clip_coef(P, P, 0, BF16, 1.0, P, P, P, None) == SHAPE
    assert lib.om_grad_norm_clip_coef(P, P, 3, BF16, 1.0, None, P, P, None) == NULL
    assert lib.om_grad_norm_clip_coef(P, P, 3, 4, 1.0, P, P, P, None) == DTYPE


def test_routers(lib):
    assert lib.om_route_softmax_topk(P, 3, 8, 64, 8, 0, P, BF16, P, None) == DTYPE
    assert lib.om_route_softmax_topk(P, F32, 8, 600, 8, 0, P, BF16, P, None) == SHAPE      # N > 512
    assert lib.om_route_softmax_topk(P, F32, 8, 4, 8, 0, P, BF16, P, None) == SHAPE        # K > N
    assert lib.om_route_softmax_topk(P, F32, 0, 64, 8, 0, P, BF16, P, None) == OK
    assert lib.om_route_softmax_topk(None, F32, 8, 64, 8, 0, P, BF16, P, None) == NULL
    assert lib.om_route_softmax_topk_bwd(P, F32, None, P, BF16, 8, 64, 8, 0, P, None) == NULL
    assert lib.om_route_sigmoid_group_topk(P, P, 8, 256, 7, 4, 8, 1, 2.5, P, P, None) == SHAPE   # 256 % 7
    assert lib.om_route_sigmoid_group_topk(P, None, 8, 256, 8, 4, 8, 1, 2.5, P, P, None) == NULL
    assert lib.om_router_gate_softmax_topk(P, P, 8, 2048, 300, 8, 0, P, P, BF16, P, None) == SHAPE   # N > 256
    assert lib.om_router_gate_softmax_topk(P, P, 8, 2000, 64, 8, 0, P, P, BF16, P, None) == SHAPE   # H % 512
    assert lib.om_router_gate_softmax_topk(ODD, P, 8, 2048, 64, 8, 0, P, P, BF16, P, None) == ALIGN
    assert lib.om_router_gate_softmax_topk(P, P, 8, 2048, 64, 8, 0, P, None, BF16, P, None) == NULL
    assert lib.om_router_gate_logits(P, P, 8, 2048, 64, None, None) == NULL
    need = lib.om_router_gate_logits_split_workspace_bytes(8192, 7168, 256)
    assert need > 0 and need % 16 == 0
    assert lib.om_router_gate_logits_split_workspace_bytes(8192, 7100, 256) == SHAPE     # H % 8
    assert lib.om_router_gate_logits_split_workspace_bytes(8192, 7168, 300) == SHAPE     # N > 256
    assert lib.om_router_gate_logits_split(P, P, 8192, 7168, 256, P, P, need - 1, None) == WORKSPACE
    assert lib.om_router_gate_logits_split(P, None, 8192, 7168, 256, P, P, need, None) == NULL
    assert lib.om_router_gate_logits_split(ODD, P, 8192, 7168, 256, P, P, need, None) == ALIGN
    assert lib.om_router_gate_logits_split(P, P, 0, 7168, 256, P, P, 0, None) == OK
    need = lib.om_router_gate_wgrad_workspace_bytes(16384, 2048, 64)
    assert need > 0 and need % 16 == 0
    assert lib.om_router_gate_wgrad_workspace_bytes(16384, 2044, 64) == SHAPE      # H % 8
    assert lib.om_router_gate_wgrad_workspace_bytes(16384, 2048, 300) == SHAPE     # more than 256 experts
    assert lib.om_router_gate_wgrad_workspace_bytes(16384, 2048, 48) > 0           # any expert count up to 256
    assert lib.om_router_gate_wgrad(P, P, 16384, 2048, 64, P, 7, P, need, None) == DTYPE
    assert lib.om_router_gate_wgrad(P, P, 16384, 2048, 0, P, BF16, P, need, None) == SHAPE
    assert lib.om_router_gate_dgrad(P, P, None, P, 16384, 2044, 64, None) == SHAPE      # H % 8
    assert lib.om_router_gate_dgrad(P, P, None, P, 16384, 2048, 257, None) == SHAPE
    assert lib.om_router_gate_dgrad(P, None, None, P, 16384, 2048, 64, None) == NULL
    assert lib.om_router_gate_dgrad(P, P, ODD, P, 16384, 2048, 64, None) == ALIGN
    assert lib.om_router_gate_dgrad(None, None, None, None, 0, 2048, 64, None) == OK
    assert lib.om_grad_scale(P, 100, 7, P, None) == DTYPE
    assert lib.om_grad_scale(P, 100, BF16, None, None) == NULL
    assert lib.om_grad_scale(ODD, 100, BF16, P, None) == ALIGN
    assert lib.om_grad_scale(None, 0, BF16, None, None) == OK
    assert lib.om_shard_clip_multiplier(P, 0, 7, 1.0, P, P, None) == DTYPE
    assert lib.om_shard_clip_multiplier(P, 2, BF16, 1.0, P, P, None) == SHAPE
    assert lib.om_shard_clip_multiplier(None, 0, BF16, 1.0, P, P, None) == NULL
    assert lib.om_shard_clip_multiplier(P, 1, BF16, 1.0, P, None, None) == NULL
    assert lib.om_adamw_traffic_probe(P, P, P, None, P, 1024, None) == NULL
    assert lib.om_router_balance_stats_masked(P, 7, P, 100, 64, 8, P, P, P, 1 << 20, None) == DTYPE
    assert lib.om_router_balance_stats_masked(P, F32, None, 100, 64, 65, P, P, P, 1 << 20, None) == SHAPE
    assert lib.om_router_balance_stats_masked(P, F32, P, 100, 64, 8, P, P, P, 8, None) == WORKSPACE
    assert lib.om_router_balance_bwd_masked(P, F32, None, P, 100, 64, P, None) == NULL
    assert lib.om_router_balance_bwd_masked(None, F32, None, None, 0, 64, None, None) == OK
    assert lib.om_router_gate_wgrad(P, P, 16384, 2048, 64, None, BF16, P, need, None) == NULL
    assert lib.om_router_gate_wgrad(P, None, 16384, 2048, 64, P, BF16, P, need, None) == NULL
    assert lib.om_router_gate_wgrad(P, P, 16384, 2048, 64, ODD, BF16, P, need, None) == ALIGN
    assert lib.om_router_gate_wgrad(P, P, 16384, 2048, 64, P, BF16, P, need - 1, None) == WORKSPACE


def test_sort_and_index_ops(lib):
    need = lib.om_moe_sort_workspace_bytes(1024, 8, 64)
    assert need > 0
    assert lib.om_moe_sort(P, 5, 1024, 8, 0, 64, P, P, P, P, P, P, need, None) == DTYPE
    assert lib.om_moe_sort(P, I64, 1024, 0, 0, 64, P, P, P, P, P, P, need, None) == SHAPE
    assert lib.om_moe_sort(P, I64, 1024, 8, 0, 64, None, P, P, P, P, P, need, None) == NULL
    assert lib.om_moe_sort(P, I64, 1024, 8, 0, 64, P, P, P, P, P, P, need - 1, None) == WORKSPACE
    assert lib.om_compute_partial_token_counts(P, I64, P, P, 0, 64, 1000, 8, 64, None) == SHAPE   # T % TH
    assert lib.om_index_gather(P, P, P, 16, 64, 3, None) == DTYPE
    assert lib.om_index_gather(P, None, P, 16, 64, BF16, None) == NULL
    assert lib.om_index_gather(P, P, P, 0, 64, BF16, None) == OK
    assert lib.om_index_add(P, P, P, -1, 64, BF16, None) == SHAPE
    assert lib.om_swiglu_fwd(P, P, ODD, 64, BF16, None) == ALIGN
    assert lib.om_swiglu_bwd(P, P, P, None, P, 64, BF16, None) == NULL


def test_rmsnorm_and_balance(lib):
    assert lib.om_rmsnorm_fwd(P, None, P, 1e-5, P, None, None, 8, 2048, 3, None) == DTYPE
    assert lib.om_rmsnorm_fwd(P, None, P, 1e-5, P, None, None, 8, 2052, BF16, None) == SHAPE   # E % 8
    assert lib.om_rmsnorm_fwd(P, None, P, 1e-5, P, None, None, 0, 2048, BF16, None) == OK
    assert lib.om_rmsnorm_fwd(P, None, None, 1e-5, P, None, None, 8, 2048, BF16, None) == NULL
    assert lib.om_rmsnorm_fwd(P, ODD, P, 1e-5, P, None, None, 8, 2048, BF16, None) == ALIGN
    need = lib.om_rmsnorm_bwd_workspace_bytes(300, 2048)
    assert need == 3 * 2048 * 4
    assert lib.om_rmsnorm_bwd(P, P, P, P, P, P, P, need - 1, 300, 2048, BF16, None) == WORKSPACE
    assert lib.om_rmsnorm_bwd(P, P, P, None, P, P, P, need, 300, 2048, BF16, None) == NULL
    need = lib.om_router_balance_workspace_bytes(1000, 64)
    assert lib.om_router_balance_stats(P, F32, 1000, 64, 8, P, P, P, need - 1, None) == WORKSPACE
    assert lib.om_router_balance_stats(P, 9, 1000, 64, 8, P, P, P, need, None) == DTYPE
    assert lib.om_router_balance_bwd(P, F32, None, 1000, 64, P, None) == NULL


def test_combine_with_residual(lib):
    args = (16384, 8, 2048, BF16, BF16, None)
    assert lib.om_reduce_ggemm_output_residual(P, P, P, P, P, None, P, *args) == NULL        # no residual
    assert lib.om_reduce_ggemm_output_residual(P, P, P, P, P, P, None, *args) == NULL
    assert lib.om_reduce_ggemm_output_residual(P, P, P, P, P, P, P, 16384, 8, 2048, 7, BF16, None) == DTYPE
    assert lib.om_reduce_ggemm_output_residual(P, P, P, P, P, None, P, 0, 8, 2048, BF16, BF16, None) == OK


def test_grouped_gemms(lib):
    args = (131072, 64, 2048, 1024, 0, None)
    assert lib.om_grouped_gemm_fwd(P, P, P, P, 131072, 64, 2004, 1024, 0, None) == SHAPE    # N % 8
    assert lib.om_grouped_gemm_fwd(P, P, P, P, 131072, 64, 2048, 1020, 0, None) == SHAPE    # K % 8
    assert lib.om_grouped_gemm_fwd(P, P, P, P, 0, 64, 2048, 1024, 0, None) == OK            # no rows
    assert lib.om_grouped_gemm_fwd(P, P, P, P, 4096, 1025, 256, 256, 0, None) == SHAPE      # G > 1024 (LDS table)
    assert lib.om_grouped_gemm_fwd(P, None, P, P, *args) == NULL
    assert lib.om_grouped_gemm_fwd(P, P, ODD, P, *args) == ALIGN
    assert lib.om_grouped_gemm_fwd(P, P, P, P, 1 << 30, 64, 2048, 1024, 0, None) == SHAPE   # 2^40 elements or more
    assert lib.om_grouped_gemm_fwd(P, P, P, P, 4096, 64, 2048, 1024, 2048 * 1024 + 4, None) == ALIGN   # expert pitch % 8
    assert lib.om_grouped_gemm_dgrad(P, P, P, None, *args) == NULL
    assert lib.om_grouped_gemm_wgrad(P, P, P, P, 131072, 0, 2048, 1024, 0, None) == SHAPE   # G < 1
    assert lib.om_merged_mlp_gate_up_fwd(P, P, P, P, P, P, P, 131072, 64, 1004, 2048, 0, None) == SHAPE
    assert lib.om_merged_mlp_gate_up_fwd(P, P, None, P, P, P, P, 131072, 64, 1024, 2048, 0, None) == NULL
    assert lib.om_merged_mlp_down_dgrad(P, P, P, P, P, ODD, P, 131072, 64, 1024, 2048, 0, None) == ALIGN
    assert lib.om_merged_mlp_gate_up_dgrad(P, P, P, P, None, P, 131072, 64, 1024, 2048, 0, None) == NULL
    # float32 forms: N, K multiples of 8
    assert lib.om_grouped_gemm_fwd_f32(P, P, P, P, 4096, 8, 100, 256, 0, None) == SHAPE
    assert lib.om_grouped_gemm_fwd_f32(P, P, P, P, 0, 8, 64, 256, 0, None) == OK
    assert lib.om_grouped_gemm_fwd_f32(P, P, P, None, 4096, 8, 64, 256, 0, None) == NULL
    assert lib.om_grouped_gemm_fwd_f32(P, P, P, P, 4096, 8, 64, 256, 64 * 256 + 2, None) == ALIGN   # pitch % 4
    assert lib.om_grouped_gemm_dgrad_f32(P, ODD, P, P, 4096, 8, 64, 256, 0, None) == ALIGN
    assert lib.om_grouped_gemm_wgrad_f32(P, P, None, P, 4096, 8, 64, 256, 0, None) == NULL
    assert lib.om_grouped_gemm_wgrad_f32(P, P, P, P, 4096, 70000, 64, 256, 0, None) == SHAPE        # grid limit
    # the forms that read the tokens through an index
    g = (131072, 64, 1024, 2048, 0, None)
    assert lib.om_merged_mlp_gate_up_fwd_gathered(P, None, 16384, P, P, P, P, P, P, *g) == NULL      # no index
    assert lib.om_merged_mlp_gate_up_fwd_gathered(P, P, 0, P, P, P, P, P, P, *g) == SHAPE            # no source rows
    assert lib.om_merged_mlp_gate_up_fwd_gathered(P, P, 1 << 20, P, P, P, P, P, P, *g) == SHAPE      # indexed source of 2^31 elements or more
    assert lib.om_merged_mlp_gate_up_fwd_gathered(P, None, 0, P, P, P, P, P, P, 0, 64, 1024, 2048, 0, None) == OK
    assert lib.om_grouped_gemm_wgrad_gathered(P, P, None, 16384, P, P, *g) == NULL
    assert lib.om_grouped_gemm_wgrad_gathered(P, P, P, 0, P, P, *g) == SHAPE
    assert lib.om_grouped_gemm_wgrad_gathered(P, P, P, 16384, ODD, P, *g) == ALIGN


def test_routing_weight_folded_into_the_expert_mlp(lib):
    g = (131072, 64, 1024, 2048, 0, None)
    assert lib.om_moe_row_weights(P, P, P, P, P, 131072, 8, 7, None) == DTYPE
    assert lib.om_moe_row_weights(P, P, P, P, None, 131072, 8, F32, None) == NULL
    assert lib.om_moe_row_weights(P, P, P, P, P, 131072, 0, F32, None) == SHAPE
    assert lib.om_moe_row_weights(None, None, None, None, None, 0, 8, BF16, None) == OK
    assert lib.om_merged_mlp_gate_up_fwd_weighted(P, P, 16384, P, P, None, P, P, P, P, *g) == NULL   # no weights
    assert lib.om_merged_mlp_gate_up_fwd_weighted(P, None, 16384, P, P, P, P, P, P, P, *g) == NULL   # no index
    assert lib.om_merged_mlp_gate_up_fwd_weighted(P, P, 0, P, P, P, P, P, P, P, *g) == SHAPE
    assert lib.om_merged_mlp_gate_up_fwd_weighted(P, P, 16384, P, P, P, P, P, P, P, 131072, 64, 1004, 2048, 0, None) == SHAPE
    assert lib.om_merged_mlp_gate_up_fwd_weighted(P, None, 0, P, P, None, P, P, P, P, 0, 64, 1024, 2048, 0, None) == OK
    assert lib.om_sum_ggemm_output(P, None, P, None, P, 16384, 2048, BF16, None) == NULL
    assert lib.om_sum_ggemm_output(P, P, P, None, P, 16384, 2048, 7, None) == DTYPE
    assert lib.om_sum_ggemm_output(P, P, P, None, P, 0, 2048, BF16, None) == OK
    gw = (131072, 64, 2048, 1024, 0, None)
    assert lib.om_grouped_gemm_wgrad_gathered_out(P, None, 16384, P, P, P, *gw) == NULL
    assert lib.om_grouped_gemm_wgrad_gathered_out(P, P, 0, P, P, P, *gw) == SHAPE
    assert lib.om_grouped_gemm_wgrad_gathered_out(P, P, 1 << 21, P, P, P, *gw) == SHAPE   # indexed source of 2^31 elements or more
    assert lib.om_grouped_gemm_wgrad_gathered_out(P, P, 16384, P, ODD, P, *gw) == ALIGN
    assert lib.om_merged_mlp_row_dot_parts(1024) == 16
    assert lib.om_merged_mlp_row_dot_parts(200) == 4      # partial last 64-column group
    assert lib.om_merged_mlp_row_dot_parts(100) == SHAPE
    assert lib.om_merged_mlp_down_dgrad_weighted(P, P, 16384, P, P, P, P, P, P, None, P, *g) == NULL   # no row_dot
    assert lib.om_merged_mlp_down_dgrad_weighted(P, P, 16384, P, P, P, None, P, P, P, P, *g) == NULL   # no weights
    assert lib.om_merged_mlp_down_dgrad_weighted(P, None, 16384, P, P, P, P, P, P, P, P, *g) == NULL   # no index
    assert lib.om_merged_mlp_down_dgrad_weighted(P, P, 0, P, P, P, P, P, P, P, P, *g) == SHAPE
    assert lib.om_merged_mlp_down_dgrad_weighted(P, P, 16384, P, P, P, P, ODD, P, P, P, *g) == ALIGN
    assert lib.om_merged_mlp_down_dgrad_weighted(P, None, 0, P, P, P, None, P, P, None, P, 0, 64, 1024, 2048, 0, None) == OK
    assert lib.om_moe_row_weights_grad(P, 0, P, P, P, P, 131072, 8, F32, None) == SHAPE
    assert lib.om_moe_row_weights_grad(None, 16, P, P, P, P, 131072, 8, F32, None) == NULL
    assert lib.om_moe_row_weights_grad(P, 16, P, P, P, P, 131072, 8, 9, None) == DTYPE
    assert lib.om_moe_row_weights_grad(None, 16, None, None, None, None, 0, 8, F32, None) == OK


def test_check_raises_with_the_library_text():
    with pytest.raises(n.NativeLibraryError, match="dtype"):
        n.check(DTYPE, "om_adamw_step")
