"""Patch rules for Mistral models: `mistral-qkvo` and `mistral-mlp` (reference:
fms_acceleration_foak/models/mistral.py).  The reference's RMSNorm / RoPE / cross-entropy rules for
this architecture belong to other kernels and are not built."""
from transformers.models.mistral.modeling_mistral import MistralAttention, MistralMLP

from ._rules import fused_lora_rules


def get_mp_rules(base_type: str, config=None):
    return fused_lora_rules("mistral", MistralAttention, MistralMLP, base_type, config, label="Mistral")
