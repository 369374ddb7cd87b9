"""Patch rules `mixtral-rms`, `mixtral-qkvo`, `mixtral-rope` (reference: fms_acceleration_foak/models/mixtral.py):
the attention projections of this mixture-of-experts architecture take the fused LoRA operators; its
expert MLPs have no fused-LoRA rule in the reference either, plus the fast cross-entropy rule
(the liger fused-linear-CE variant is not built)."""
from transformers.models.mixtral.modeling_mixtral import MixtralAttention, MixtralForCausalLM, MixtralRMSNorm

from ._rules import fused_lora_rules, loss_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None):
    return [
        *fused_lora_rules("mixtral", MixtralAttention, None, base_type, config, label="Mixtral"),
        *loss_rules("mixtral", MixtralForCausalLM, "transformers.models.mixtral.modeling_mixtral"),
        *norm_rope_rules("mixtral", MixtralRMSNorm, "transformers.models.mixtral.modeling_mixtral"),
    ]
