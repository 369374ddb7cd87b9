"""Patch rules for Llama models: `llama-rms`, `llama-qkvo`, `llama-mlp`, `llama-rope` (reference:
fms_acceleration_foak/models/llama.py).  The reference's cross-entropy rules for this architecture
belong to other kernels and are not built."""
from transformers.models.llama.modeling_llama import LlamaAttention, LlamaMLP, LlamaRMSNorm

from ._rules import fused_lora_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None):
    return [
        *fused_lora_rules("llama", LlamaAttention, LlamaMLP, base_type, config, label="Llama"),
        *norm_rope_rules("llama", LlamaRMSNorm, "transformers.models.llama.modeling_llama"),
    ]
