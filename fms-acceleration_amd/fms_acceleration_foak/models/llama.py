"""Patch rules for Llama models: `llama-qkvo` and `llama-mlp` (reference:
fms_acceleration_foak/models/llama.py).  The reference's RMSNorm / RoPE / cross-entropy rules for
this architecture belong to other kernels and are not built."""
from transformers.models.llama.modeling_llama import LlamaAttention, LlamaMLP

from ._rules import fused_lora_rules


def get_mp_rules(base_type: str, config=None):
    return fused_lora_rules("llama", LlamaAttention, LlamaMLP, base_type, config, label="Llama")
