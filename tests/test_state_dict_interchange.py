"""Merged <-> per-expert checkpoint key mapping (reference generate_parallel_model.py:136-148 and
evals/convert_olmoe_om_checkpoint_to_hf.py:59-88).  Host logic only."""
import pytest
import torch

from optimus.models.common.moe import merged_state_dict_to_per_expert, per_expert_state_dict_to_merged


def _serial(num_experts=8, I=6, H=4):
    g = torch.Generator().manual_seed(0)
    sd = {"model.layers.3.mlp.gate.weight": torch.randn(num_experts, H, generator=g),
          "model.layers.3.input_layernorm.weight": torch.randn(H, generator=g)}
    for e in range(num_experts):
        p = f"model.layers.3.mlp.experts.{e}"
        sd[f"{p}.gate_proj.weight"] = torch.randn(I, H, generator=g)
        sd[f"{p}.up_proj.weight"] = torch.randn(I, H, generator=g)
        sd[f"{p}.down_proj.weight"] = torch.randn(H, I, generator=g)
    return sd


def test_round_trip_whole_model():
    sd = _serial()
    merged = per_expert_state_dict_to_merged(sd, 8)
    assert merged["model.layers.3.mlp.experts.gate_proj_merged_weight"].shape == (8, 6, 4)
    assert merged["model.layers.3.mlp.experts.down_proj_merged_weight"].shape == (8, 4, 6)
    assert not any(".experts.0." in k for k in merged)
    back = merged_state_dict_to_per_expert(merged)
    assert back.keys() == sd.keys() and all(torch.equal(back[k], sd[k]) for k in sd)


def test_expert_parallel_window_uses_global_ids():
    sd = _serial()
    merged = per_expert_state_dict_to_merged(sd, num_local_experts=2, expert_start_id=4)   # rank 2 of 4
    w = merged["model.layers.3.mlp.experts.up_proj_merged_weight"]
    assert w.shape[0] == 2 and torch.equal(w[1], sd["model.layers.3.mlp.experts.5.up_proj.weight"])
    back = merged_state_dict_to_per_expert(merged, expert_start_id=4)
    assert "model.layers.3.mlp.experts.4.gate_proj.weight" in back
    assert "model.layers.3.mlp.experts.0.gate_proj.weight" not in back
    # un-merging hands out views of the merged tensor, not copies
    assert back["model.layers.3.mlp.experts.5.up_proj.weight"].data_ptr() == w[1].data_ptr()


def test_missing_expert_is_an_error():
    sd = _serial()
    del sd["model.layers.3.mlp.experts.6.down_proj.weight"]
    with pytest.raises(KeyError, match="6"):
        per_expert_state_dict_to_merged(sd, 8)


def test_merged_keys_load_into_the_merged_module():
    from optimus.models.common.moe import MergedMLP
    from optimus.models.olmoe.configuration_olmoe import OlmoeParallelConfig
    cfg = OlmoeParallelConfig(hidden_size=4, intermediate_size=6, num_experts=8)
    mlp = MergedMLP(cfg)
    merged = per_expert_state_dict_to_merged(_serial(), 8)
    prefix = "model.layers.3.mlp.experts."
    mlp.load_state_dict({k[len(prefix):]: v for k, v in merged.items() if k.startswith(prefix)})
    assert torch.equal(mlp.gate_proj_merged_weight[3], _serial()["model.layers.3.mlp.experts.3.gate_proj.weight"])
