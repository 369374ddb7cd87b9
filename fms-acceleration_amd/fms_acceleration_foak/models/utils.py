"""Builders of the patched forwards (reference: fms_acceleration_foak/models/utils.py).

`FUSED_OPS[base_type][key]` is the operator table the patch rules draw from; q/k/v share one fused
call through a small per-attention cache: the first of the three projections to be called with X
runs the fused operator, each projection then pops its own output (:60-100 of the reference).
"""
from __future__ import annotations

from functools import partial
from typing import Callable, List, Type

import torch

from fms_acceleration.model_patcher import ModelPatcherTrigger

from ..fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_mlp_swiglu as fused_op_mlp_bnb
from ..fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_o_v2 as fused_op_o_bnb
from ..fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_qkv as fused_op_qkv_bnb
from ..fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_mlp as fused_op_mlp_gptq
from ..fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_o_v2 as fused_op_o_gptq
from ..fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_qkv as fused_op_qkv_gptq

KEY_QKV = "qkv"
KEY_O = "o"
KEY_MLP = "mlp"

KEY_HIDDEN_ACTIVATIONS = ["hidden_act", "activation_function"]

FUSED_OPS = {
    "auto_gptq": {KEY_QKV: fused_op_qkv_gptq, KEY_O: fused_op_o_gptq, KEY_MLP: fused_op_mlp_gptq},
    "bitsandbytes": {KEY_QKV: fused_op_qkv_bnb, KEY_O: fused_op_o_bnb, KEY_MLP: fused_op_mlp_bnb},
}


def register_fused_ops(base_type: str, qkv: Callable, o: Callable, mlp: Callable):
    FUSED_OPS[base_type] = {KEY_QKV: qkv, KEY_O: o, KEY_MLP: mlp}


def _is_loralayer(module: torch.nn.Module, names: List[str] = None):
    """Duck-typed LoRA-layer test (:46-49)."""
    names = names or ["lora_A", "lora_B", "base_layer"]
    return all(hasattr(module, n) for n in names)


def _build_fused_forwards(attn: torch.nn.Module, fused_operation: Callable, submodule_names: List[str]):
    """One closure per sub-module name.  Protocol: each of the named projections is called exactly
    once per attention forward; the first call computes all outputs.  Not thread-safe."""
    pending = {}

    def _forward(self, X, name: str):
        if not any(n in pending for n in submodule_names):
            outs = fused_operation(attn, X)
            outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
            pending.update(zip(submodule_names, outs))
        assert name in pending, "Fused_op needs to be first reset with sequential calls to each of them"
        return pending.pop(name)

    return [(n, partial(_forward, name=n)) for n in submodule_names]


def build_lora_fused_ops(attn: torch.nn.Module, base_type: str = "auto_gptq", submodule_names: List[str] = None,
                         fused_op: str = KEY_QKV):
    assert submodule_names is None or len(submodule_names) > 0, \
        "When building lora fused ops requires more than one submodule."
    if submodule_names is None:
        submodule_names = ["q_proj", "k_proj", "v_proj"]
    fused_operation = FUSED_OPS[base_type][fused_op]
    if fused_op == KEY_QKV:
        return [
            (ModelPatcherTrigger(check=_is_loralayer, module_name=name), forward)
            for name, forward in _build_fused_forwards(attn, fused_operation, submodule_names)
        ]
    if fused_op == KEY_O:
        return [(ModelPatcherTrigger(check=_is_loralayer, module_name=submodule_names[0]), fused_operation)]
    if fused_op == KEY_MLP:
        return fused_operation  # bound on the MLP module itself
    raise NotImplementedError(f"Unknown fused op '{fused_op}'")


def trigger_fused_ops(module: torch.nn.Module, attn_cls: Type, submodule_names: List[str]):
    """Module is of the attention / MLP class and every named child is a LoRA layer.  A missing
    child raises AttributeError, which the trigger treats as 'not triggered'."""
    children = [getattr(module, n) for n in submodule_names]
    return isinstance(module, attn_cls) and all(_is_loralayer(c) for c in children)


def get_hidden_activation_fn_key(config):
    for key in KEY_HIDDEN_ACTIVATIONS:
        value = getattr(config, key, None)
        if value:
            return value
    raise ValueError(f"Unable to determine activation function key for architecture {config.architectures}.")
