"""Patch rules `granitemoehybrid-rms`, `granitemoehybrid-qkvo`, `granitemoehybrid-rope` (reference: fms_acceleration_foak/models/granitemoehybrid.py):
the attention projections of this mixture-of-experts architecture take the fused LoRA operators; its
expert MLPs have no fused-LoRA rule in the reference either, plus the fast cross-entropy rule
(the liger fused-linear-CE variant is not built)."""
from transformers.models.granitemoehybrid.modeling_granitemoehybrid import GraniteMoeHybridAttention, GraniteMoeHybridForCausalLM, GraniteMoeHybridRMSNorm

from ._rules import fused_lora_rules, loss_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None):
    return [
        *fused_lora_rules("granitemoehybrid", GraniteMoeHybridAttention, None, base_type, config, label="GraniteMoeHybrid"),
        *loss_rules("granitemoehybrid", GraniteMoeHybridForCausalLM, "transformers.models.granitemoehybrid.modeling_granitemoehybrid"),
        *norm_rope_rules("granitemoehybrid", GraniteMoeHybridRMSNorm, "transformers.models.granitemoehybrid.modeling_granitemoehybrid"),
    ]
