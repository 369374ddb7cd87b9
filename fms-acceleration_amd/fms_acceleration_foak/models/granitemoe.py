"""Patch rules `granitemoe-rms`, `granitemoe-qkvo`, `granitemoe-rope` (reference: fms_acceleration_foak/models/granitemoe.py):
the attention projections of this mixture-of-experts architecture take the fused LoRA operators; its
expert MLPs have no fused-LoRA rule in the reference either, plus the fast cross-entropy rule
(the liger fused-linear-CE variant is not built)."""
from transformers.models.granitemoe.modeling_granitemoe import GraniteMoeAttention, GraniteMoeForCausalLM, GraniteMoeRMSNorm

from ._rules import fused_lora_rules, loss_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None):
    return [
        *fused_lora_rules("granitemoe", GraniteMoeAttention, None, base_type, config, label="GraniteMoe"),
        *loss_rules("granitemoe", GraniteMoeForCausalLM, "transformers.models.granitemoe.modeling_granitemoe"),
        *norm_rope_rules("granitemoe", GraniteMoeRMSNorm, "transformers.models.granitemoe.modeling_granitemoe"),
    ]
