"""Patch rules for Granite models: `granite-rms`, `granite-qkvo`, `granite-mlp`, `granite-rope` (reference:
fms_acceleration_foak/models/granite.py).  The reference's cross-entropy rules for this architecture
belong to other kernels and are not built."""
from transformers.models.granite.modeling_granite import GraniteAttention, GraniteMLP, GraniteRMSNorm

from ._rules import fused_lora_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None):
    return [
        *fused_lora_rules("granite", GraniteAttention, GraniteMLP, base_type, config, label="Granite"),
        *norm_rope_rules("granite", GraniteRMSNorm, "transformers.models.granite.modeling_granite"),
    ]
