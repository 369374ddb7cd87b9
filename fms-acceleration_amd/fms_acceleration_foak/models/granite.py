"""Patch rules for Granite models: `granite-qkvo` and `granite-mlp` (reference:
fms_acceleration_foak/models/granite.py).  The reference's RMSNorm / RoPE / cross-entropy rules for
this architecture belong to other kernels and are not built."""
from transformers.models.granite.modeling_granite import GraniteAttention, GraniteMLP

from ._rules import fused_lora_rules


def get_mp_rules(base_type: str, config=None):
    return fused_lora_rules("granite", GraniteAttention, GraniteMLP, base_type, config, label="Granite")
