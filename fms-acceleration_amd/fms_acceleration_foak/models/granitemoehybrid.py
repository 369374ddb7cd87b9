"""Patch rule `granitemoehybrid-qkvo` (reference: fms_acceleration_foak/models/granitemoehybrid.py): the attention
projections of this mixture-of-experts architecture take the fused LoRA operators; its expert MLPs
have no fused-LoRA rule in the reference either, and its RMSNorm / RoPE / loss rules belong to
other kernels and are not built."""
from transformers.models.granitemoehybrid.modeling_granitemoehybrid import GraniteMoeHybridAttention

from ._rules import fused_lora_rules


def get_mp_rules(base_type: str, config=None):
    return fused_lora_rules("granitemoehybrid", GraniteMoeHybridAttention, None, base_type, config, label="GraniteMoeHybrid")
