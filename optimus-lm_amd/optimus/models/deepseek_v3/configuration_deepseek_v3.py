"""DeepseekV3ParallelConfig — same constructor keywords and defaults as the reference
(optimus/models/deepseek_v3/configuration_deepseek_v3.py:4-37); the MoE block reads
hidden_size, moe_intermediate_size, n_shared_experts, n_routed_experts, routed_scaling_factor,
n_group, topk_group, num_experts_per_tok, norm_topk_prob and the parallelism fields."""


class DeepseekV3ParallelConfig():
    def __init__(self, vocab_size=129280, hidden_size=7168, intermediate_size=18432,
                 moe_intermediate_size=2048, num_hidden_layers=61, num_attention_heads=128,
                 n_shared_experts=1, n_routed_experts=256, routed_scaling_factor=2.5,
                 kv_lora_rank=512, q_lora_rank=1536, qk_rope_head_dim=64, v_head_dim=128,
                 qk_nope_head_dim=128, n_group=8, topk_group=4, num_experts_per_tok=8,
                 first_k_dense_replace=3, norm_topk_prob=True, max_position_embeddings=4096,
                 initializer_range=0.02, rms_norm_eps=1e-6, rope_interleave=True, pad_token_id=None,
                 expert_parallelism=1, pipeline_parallelism=1, tensor_parallelism=1,
                 virtual_pipeline_parallelism=1, use_activation_checkpointing=False,
                 activation_checkpointing_level=0, force_uniform_routing=False):
        values = dict(locals())
        values.pop("self")
        for k, v in values.items():
            setattr(self, k, v)
        self.head_dim = self.qk_rope_head_dim
        self.num_key_value_heads = self.num_attention_heads
        self.qk_head_dim = self.qk_nope_head_dim + self.qk_rope_head_dim
        self.attention_bias = False
        self.attention_dropout = 0.0
        self.rope_theta = 10000
        self.use_cache = False

    def __repr__(self):
        lines = ['DeepseekV3ParallelConfig : {']
        for k, v in self.__dict__.items():
            lines.append(f'    "{k}": {repr(v)},')
        lines.append('}')
        return "\n".join(lines)

    __str__ = __repr__
