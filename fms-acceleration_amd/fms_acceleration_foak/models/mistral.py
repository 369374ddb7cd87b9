"""Patch rules for Mistral models: `mistral-rms`, `mistral-qkvo`, `mistral-mlp`, `mistral-rope` (reference:
fms_acceleration_foak/models/mistral.py).  The reference's cross-entropy rules for this architecture
belong to other kernels and are not built."""
from transformers.models.mistral.modeling_mistral import MistralAttention, MistralMLP, MistralRMSNorm

from ._rules import fused_lora_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None):
    return [
        *fused_lora_rules("mistral", MistralAttention, MistralMLP, base_type, config, label="Mistral"),
        *norm_rope_rules("mistral", MistralRMSNorm, "transformers.models.mistral.modeling_mistral"),
    ]
