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

from ..fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_qkv_rope as fused_op_qkv_rope_bnb
from ..fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_qkv_rope as fused_op_qkv_rope_gptq

KEY_QKV = "qkv"
KEY_O = "o"
KEY_MLP = "mlp"

KEY_HIDDEN_ACTIVATIONS = ["hidden_act", "activation_function"]

FUSED_OPS = {
    "auto_gptq": {KEY_QKV: fused_op_qkv_gptq, KEY_O: fused_op_o_gptq, KEY_MLP: fused_op_mlp_gptq},
    "bitsandbytes": {KEY_QKV: fused_op_qkv_bnb, KEY_O: fused_op_o_bnb, KEY_MLP: fused_op_mlp_bnb},
}


# Q / K / V with the rotary embedding of Q and K applied inside the projection launch (no counterpart in the reference,
# whose fused projections are followed by the separate fast_rope_embedding pass); chosen by `qkv_rope` below
FUSED_QKV_ROPE_OPS = {"auto_gptq": fused_op_qkv_rope_gptq, "bitsandbytes": fused_op_qkv_rope_bnb}


def register_fused_ops(base_type: str, qkv: Callable, o: Callable, mlp: Callable):
    FUSED_OPS[base_type] = {KEY_QKV: qkv, KEY_O: o, KEY_MLP: mlp}


def _is_loralayer(module: torch.nn.Module, names: List[str] = None):
    """Duck-typed LoRA-layer test (:46-49)."""
    names = names or ["lora_A", "lora_B", "base_layer"]
    return all(hasattr(module, n) for n in names)


def _build_fused_forwards(attn: torch.nn.Module, fused_operation: Callable, submodule_names: List[str],
                          rope_operation: Callable = None):
    """One closure per sub-module name.  Protocol: each of the named projections is called exactly
    once per attention forward; the first call computes all outputs.  Not thread-safe.

    rope_operation (apply_lora_qkv_rope): a forward pre-hook of the attention keeps the `position_embeddings` it is
    called with; the fused call then returns Q and K already rotated and marks them, so that the attention's
    apply_rotary_pos_emb (fast_rope_embedding of the `<arch>-rope` rule) passes them through.  Without tables
    (an attention called without `position_embeddings`) the plain fused operation runs.  A forward hook that runs
    whether or not the forward raised closes the protocol: a mark that is still there when the attention returns
    means its rotation did not go through fast_rope_embedding (Q / K would leave rotated twice), which raises at
    once; after an exception inside the forward the mark and the pending outputs are dropped, so a retry starts clean."""
    pending = {}
    tables = {}

    if rope_operation is not None:
        from ..kernels.unsloth.rope_embedding import mark_rotated, unmark_rotated  # pylint: disable=import-outside-toplevel

        def _keep_tables(module, args, kwargs):
            tables["pe"] = kwargs.get("position_embeddings", args[1] if len(args) > 1 else None)

        def _close_protocol(module, args, output):
            key = tables.pop("marked", None)
            tables.pop("pe", None)
            unconsumed = key is not None and unmark_rotated(key)
            if output is None:  # the forward raised: leave nothing behind for the next call
                pending.clear()
                return
            if unconsumed:
                raise RuntimeError("fused Q/K/V with rotary embedding: the attention returned without handing the rotated "
                                   "Q / K to apply_rotary_pos_emb (fast_rope_embedding): its outputs are rotated twice; "
                                   "enable fast_rope_embeddings for this model or switch the fused rotation off")

        attn.register_forward_pre_hook(_keep_tables, with_kwargs=True)
        attn.register_forward_hook(_close_protocol, always_call=True)

    def _forward(self, X, name: str):
        if not any(n in pending for n in submodule_names):
            pe = tables.pop("pe", None)
            if rope_operation is not None and pe is not None and X.dim() == 3:
                outs = rope_operation(attn, X, pe[0], pe[1])
                tables["marked"] = mark_rotated(outs[0], outs[1])
            else:
                outs = fused_operation(attn, X)
            outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
            pending.update(zip(submodule_names, outs))
        assert name in pending, "Fused_op needs to be first reset with sequential calls to each of them"
        return pending.pop(name)

    return [(n, partial(_forward, name=n)) for n in submodule_names]


def build_lora_fused_ops(attn: torch.nn.Module, base_type: str = "auto_gptq", submodule_names: List[str] = None,
                         fused_op: str = KEY_QKV, qkv_rope: bool = False):
    assert submodule_names is None or len(submodule_names) > 0, \
        "When building lora fused ops requires more than one submodule."
    if submodule_names is None:
        submodule_names = ["q_proj", "k_proj", "v_proj"]
    fused_operation = FUSED_OPS[base_type][fused_op]
    if fused_op == KEY_QKV:
        return [
            (ModelPatcherTrigger(check=_is_loralayer, module_name=name), forward)
            for name, forward in _build_fused_forwards(attn, fused_operation, submodule_names,
                                                       FUSED_QKV_ROPE_OPS.get(base_type) if qkv_rope else None)
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
