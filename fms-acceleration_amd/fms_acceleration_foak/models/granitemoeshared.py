"""Patch rules `granitemoeshared-rms`, `granitemoeshared-qkvo`, `granitemoeshared-rope` (reference: fms_acceleration_foak/models/granitemoeshared.py):
the attention projections of this mixture-of-experts architecture take the fused LoRA operators; its
expert MLPs have no fused-LoRA rule in the reference either, plus the fast cross-entropy rule
(the liger fused-linear-CE variant is not built)."""
from transformers.models.granitemoeshared.modeling_granitemoeshared import GraniteMoeSharedAttention, GraniteMoeSharedForCausalLM, GraniteMoeSharedRMSNorm

from ._rules import fused_lora_rules, loss_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None):
    return [
        *fused_lora_rules("granitemoeshared", GraniteMoeSharedAttention, None, base_type, config, label="GraniteMoeShared"),
        *loss_rules("granitemoeshared", GraniteMoeSharedForCausalLM, "transformers.models.granitemoeshared.modeling_granitemoeshared"),
        *norm_rope_rules("granitemoeshared", GraniteMoeSharedRMSNorm, "transformers.models.granitemoeshared.modeling_granitemoeshared"),
    ]
