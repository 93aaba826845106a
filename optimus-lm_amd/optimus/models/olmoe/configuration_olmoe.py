"""OlmoeParallelConfig — plain-attribute config, same constructor keywords and defaults as the
reference (optimus/models/olmoe/configuration_olmoe.py:4-85).  Only the attributes the MoE block
reads matter to this build; the others are carried so existing call sites keep working."""


class OlmoeParallelConfig():
    def __init__(self, vocab_size=50304, hidden_size=2048, intermediate_size=1024,
                 num_hidden_layers=16, num_attention_heads=16, num_key_value_heads=None,
                 rms_norm_eps=1e-05, max_position_embeddings=4096, initializer_range=0.02,
                 padding_idx=1, rope_scaling=None, rope_theta=10000.0, num_experts=64,
                 num_experts_per_tok=8, norm_topk_prob=False, router_aux_loss_coef=0.01,
                 output_router_logits=False, use_local_router_aux_loss=False, use_cache=False,
                 pipeline_parallelism=1, expert_parallelism=1, tensor_parallelism=1,
                 virtual_pipeline_parallelism=1, use_activation_checkpointing=False,
                 activation_checkpointing_level=0, use_fast_moe=False,
                 use_merged_mlp_in_fast_moe=False, use_triton_path_for_gemm_in_fast_moe=False,
                 use_triton_path_for_nongemm_in_fast_moe=False, clip_qkv=None, use_qk_norm=True,
                 skip_qk_norm=False, force_uniform_routing=False):
        values = dict(locals())
        values.pop("self")
        if values["num_key_value_heads"] is None:
            values["num_key_value_heads"] = num_attention_heads
        for k, v in values.items():
            setattr(self, k, v)
        assert self.num_attention_heads % self.num_key_value_heads == 0

    def check_compatibility(self):
        assert (self.num_hidden_layers % self.pipeline_parallelism) == 0
        assert (self.num_experts % self.expert_parallelism) == 0, \
            f"num_experts {self.num_experts} should be divisible by expert_parallelism {self.expert_parallelism}"
        assert (self.tensor_parallelism == 1)

    def __repr__(self):
        lines = ['OlmoeParallelConfig : {']
        for k, v in self.__dict__.items():
            lines.append(f'    "{k}": {repr(v)},')
        lines.append('}')
        return "\n".join(lines)

    __str__ = __repr__


__all__ = ["OlmoeParallelConfig"]
