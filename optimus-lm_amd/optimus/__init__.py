"""MI355X-native implementation of Optimus-LM's single-GPU MoE + AdamW hot path.

Mirrors the reference's `optimus` namespace for the modules on that path:
optimus.custom_ops, optimus.optimizers, optimus.models.common.moe,
optimus.models.olmoe, optimus.models.deepseek_v3 (MoE parts), optimus.profilers.
All compute goes through liboptimus_mi355x.so (see optimus._native).
"""
