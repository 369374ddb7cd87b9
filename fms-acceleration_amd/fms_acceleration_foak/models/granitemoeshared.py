"""Patch rules `granitemoeshared-rms`, `granitemoeshared-qkvo`, `granitemoeshared-rope` (reference: fms_acceleration_foak/models/granitemoeshared.py):
the attention projections of this mixture-of-experts architecture take the fused LoRA operators; its
expert MLPs have no fused-LoRA rule in the reference either, and its loss rules belong to other
kernels and are not built."""
from transformers.models.granitemoeshared.modeling_granitemoeshared import GraniteMoeSharedAttention, GraniteMoeSharedRMSNorm

from ._rules import fused_lora_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None):
    return [
        *fused_lora_rules("granitemoeshared", GraniteMoeSharedAttention, None, base_type, config, label="GraniteMoeShared"),
        *norm_rope_rules("granitemoeshared", GraniteMoeSharedRMSNorm, "transformers.models.granitemoeshared.modeling_granitemoeshared"),
    ]
