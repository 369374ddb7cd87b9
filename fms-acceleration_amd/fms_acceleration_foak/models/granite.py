"""Patch rules for Granite models: `granite-rms`, `granite-qkvo`, `granite-mlp`, `granite-rope` (reference:
fms_acceleration_foak/models/granite.py).  Plus the loss rules: `granite-custom-loss` /
`granite-cross-ent` (fast cross entropy) and `granite-fused-lce` (lm_head matmul fused with the loss)."""
from transformers.models.granite.modeling_granite import GraniteAttention, GraniteForCausalLM, GraniteMLP, GraniteRMSNorm

from ._rules import fused_lce_rules, fused_lora_rules, loss_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None, qkv_rope: bool = False):
    return [
        *fused_lora_rules("granite", GraniteAttention, GraniteMLP, base_type, config, label="Granite", qkv_rope=qkv_rope),
        *fused_lce_rules("granite", GraniteForCausalLM),
        *loss_rules("granite", GraniteForCausalLM, "transformers.models.granite.modeling_granite"),
        *norm_rope_rules("granite", GraniteRMSNorm, "transformers.models.granite.modeling_granite"),
    ]
