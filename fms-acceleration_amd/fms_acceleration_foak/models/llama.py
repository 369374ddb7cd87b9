"""Patch rules for Llama models: `llama-rms`, `llama-qkvo`, `llama-mlp`, `llama-rope` (reference:
fms_acceleration_foak/models/llama.py).  Plus the loss rules: `llama-custom-loss` /
`llama-cross-ent` (fast cross entropy) and `llama-fused-lce` (lm_head matmul fused with the loss)."""
from transformers.models.llama.modeling_llama import LlamaAttention, LlamaForCausalLM, LlamaMLP, LlamaRMSNorm

from ._rules import fused_lce_rules, fused_lora_rules, loss_rules, norm_rope_rules


def get_mp_rules(base_type: str, config=None, qkv_rope: bool = False):
    return [
        *fused_lora_rules("llama", LlamaAttention, LlamaMLP, base_type, config, label="Llama", qkv_rope=qkv_rope),
        *fused_lce_rules("llama", LlamaForCausalLM),
        *loss_rules("llama", LlamaForCausalLM, "transformers.models.llama.modeling_llama"),
        *norm_rope_rules("llama", LlamaRMSNorm, "transformers.models.llama.modeling_llama"),
    ]
