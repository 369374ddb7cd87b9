"""Patch rule `granitemoeshared-qkvo` (reference: fms_acceleration_foak/models/granitemoeshared.py): the attention
projections of this mixture-of-experts architecture take the fused LoRA operators; its expert MLPs
have no fused-LoRA rule in the reference either, and its RMSNorm / RoPE / loss rules belong to
other kernels and are not built."""
from transformers.models.granitemoeshared.modeling_granitemoeshared import GraniteMoeSharedAttention

from ._rules import fused_lora_rules


def get_mp_rules(base_type: str, config=None):
    return fused_lora_rules("granitemoeshared", GraniteMoeSharedAttention, None, base_type, config, label="GraniteMoeShared")
