"""Patch rules for Mistral models: `mistral-rms`, `mistral-qkvo`, `mistral-mlp`, `mistral-rope` (reference:
fms_acceleration_foak/models/mistral.py).  Plus the loss rules: `mistral-custom-loss` /
`mistral-cross-ent` (fast cross entropy) and `mistral-fused-lce` (lm_head matmul fused with the loss)."""
from transformers.models.mistral.modeling_mistral import MistralAttention, MistralForCausalLM, MistralMLP, MistralRMSNorm

from ._rules import fused_lce_rules, fused_lora_rules, loss_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None, qkv_rope: bool = False):
    return [
        *fused_lora_rules("mistral", MistralAttention, MistralMLP, base_type, config, label="Mistral", qkv_rope=qkv_rope),
        *fused_lce_rules("mistral", MistralForCausalLM),
        *loss_rules("mistral", MistralForCausalLM, "transformers.models.mistral.modeling_mistral"),
        *norm_rope_rules("mistral", MistralRMSNorm, "transformers.models.mistral.modeling_mistral"),
    ]
