"""Shared construction of the patch rules: `<arch>-qkvo` / `<arch>-mlp` (fused LoRA; the
architectures differ only in their attention / MLP classes, reference models/llama.py:73-123,
mistral.py:70-119, granite.py:78-128), `<arch>-rms` (RMS layer norm forward replaced, llama.py:65-69)
`<arch>-rope` (the modelling module's apply_rotary_pos_emb replaced, llama.py:154-161) and the loss
rule (`<arch>-custom-loss` on transformers >= 4.46, else `<arch>-cross-ent`, llama.py:129-149)."""
from __future__ import annotations

import warnings
from functools import partial

from fms_acceleration.model_patcher import (
    ModelPatcherRule,
    ModelPatcherTrigger,
    combine_functions,
    combine_triggers,
)

from ..utils import filter_mp_rules
from .utils import KEY_MLP, KEY_O, KEY_QKV, build_lora_fused_ops, get_hidden_activation_fn_key, trigger_fused_ops

QKV_NAMES = ["q_proj", "k_proj", "v_proj"]
MLP_NAMES = ["up_proj", "down_proj", "gate_proj"]


def fused_lora_rules(arch: str, attn_cls, mlp_cls, base_type: str, config=None, label: str = None, qkv_rope: bool = False):
    """qkv_rope: the fused Q / K / V call also applies the rotary embedding (needs the `<arch>-rope` rule, whose
    fast_rope_embedding passes the marked Q / K through)."""
    rules = [
        ModelPatcherRule(
            rule_id=f"{arch}-qkvo",
            trigger=combine_triggers(
                ModelPatcherTrigger(check=partial(trigger_fused_ops, attn_cls=attn_cls, submodule_names=QKV_NAMES)),
                ModelPatcherTrigger(check=partial(trigger_fused_ops, attn_cls=attn_cls, submodule_names=["o_proj"])),
                logic="OR",
            ),
            forward_builder=combine_functions(
                partial(build_lora_fused_ops, submodule_names=QKV_NAMES, fused_op=KEY_QKV, base_type=base_type,
                        qkv_rope=qkv_rope),
                partial(build_lora_fused_ops, submodule_names=["o_proj"], fused_op=KEY_O, base_type=base_type),
                logic="APPEND",
            ),
        ),
    ]
    if mlp_cls is not None:
        rules.append(
            ModelPatcherRule(
                rule_id=f"{arch}-mlp",
                trigger=ModelPatcherTrigger(check=partial(trigger_fused_ops, attn_cls=mlp_cls, submodule_names=MLP_NAMES)),
                forward_builder=partial(build_lora_fused_ops, submodule_names=MLP_NAMES, fused_op=KEY_MLP,
                                        base_type=base_type),
            )
        )
    # only SwiGLU is fused: any other activation drops the MLP rule (llama.py:164-172)
    if config is not None and mlp_cls is not None:
        act = get_hidden_activation_fn_key(config)
        if act != "silu":
            warnings.warn(
                f"{label or arch}Rules: activation is {act}, thus disabling LoRA fused-op for MLP, since only "
                "SwiGLU is supported. This only affects quantized-peft."
            )
            rules = filter_mp_rules(rules, {"mlp"}, drop=True)
    return rules


def norm_rope_rules(arch: str, rms_cls, modeling_module: str):
    """`<arch>-rms` and `<arch>-rope` on the libfmsa_hip kernels."""
    from ..kernels.unsloth import fast_rms_layernorm, fast_rope_embedding  # pylint: disable=import-outside-toplevel

    return [
        ModelPatcherRule(rule_id=f"{arch}-rms", trigger=ModelPatcherTrigger(check=rms_cls), forward=fast_rms_layernorm),
        ModelPatcherRule(
            rule_id=f"{arch}-rope",
            import_and_maybe_reload=(f"{modeling_module}.apply_rotary_pos_emb", fast_rope_embedding, None),
        ),
    ]


def loss_rules(arch: str, causal_lm_cls, modeling_module: str):
    """The fast cross-entropy rule: newer transformers route the loss through `model.loss_function`
    (LOSS_MAPPING), older ones instantiate torch.nn.CrossEntropyLoss inside the modelling module."""
    import transformers  # pylint: disable=import-outside-toplevel
    from packaging.version import Version  # pylint: disable=import-outside-toplevel

    from ..kernels.unsloth import FastCrossEntropyLoss, replace_custom_loss_when_triggered  # pylint: disable=import-outside-toplevel

    if Version(transformers.__version__) >= Version("4.46"):
        return [
            ModelPatcherRule(
                rule_id=f"{arch}-custom-loss",
                trigger=ModelPatcherTrigger(check=replace_custom_loss_when_triggered(causal_lm_cls, custom_loss_type=f"{arch}-custom-loss")),
            )
        ]
    return [
        ModelPatcherRule(
            rule_id=f"{arch}-cross-ent",
            import_and_maybe_reload=("torch.nn.CrossEntropyLoss", FastCrossEntropyLoss, modeling_module),
        )
    ]


def fused_lce_rules(arch: str, causal_lm_cls):
    """`<arch>-fused-lce`: the causal-LM forward with the lm_head matmul and the loss fused."""
    from ..fused_ops.liger_ce import lce_forward  # pylint: disable=import-outside-toplevel

    return [ModelPatcherRule(rule_id=f"{arch}-fused-lce", trigger=ModelPatcherTrigger(check=causal_lm_cls), forward=lce_forward)]
