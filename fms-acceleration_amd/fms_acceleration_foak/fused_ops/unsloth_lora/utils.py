"""bitsandbytes-flavoured helpers of the fused operators (reference:
fused_ops/unsloth_lora/utils.py:53-141, 250-283): quant-state lookup, parameter scrape, and
`fast_dequantize`, which here is one launch of libfmsa_hip's NF4 kernel instead of two ctypes calls
into libbitsandbytes."""
from __future__ import annotations

import torch

import fmsa_hip


def QUANT_STATE(W, base_layer):
    """The quant state normally rides on the weight; fall back to the layer (FSDP re-creates the
    parameter and drops python attributes)."""
    if hasattr(W, "quant_state"):
        return W.quant_state
    return getattr(base_layer, "quant_state", None)


def get_lora_parameters(proj):
    base_layer = proj.base_layer if hasattr(proj, "base_layer") else proj
    W = base_layer.weight
    bias = base_layer.bias if hasattr(base_layer, "bias") else None
    if not hasattr(proj, "disable_adapters") or proj.disable_adapters or proj.merged:
        return W, QUANT_STATE(W, base_layer), bias, None, None, None, None
    active = proj.active_adapters[0] if hasattr(proj, "active_adapters") else proj.active_adapter
    A = proj.lora_A[active].weight
    B = proj.lora_B[active].weight
    s = proj.scaling[active]
    dropout = proj.lora_dropout[active] if hasattr(proj, "lora_dropout") else None
    return W, QUANT_STATE(W, base_layer), bias, A, B, s, dropout


def fast_dequantize(W, quant_state=None, out_dtype=None):
    """Dense weight of an NF4 tensor with double-quantised absmax, as [N, K] row-major (callers
    transpose the view when they need [K, N]).  Without a quant state W is returned as is."""
    if quant_state is None:
        return W
    from fmsa_hip.nf4_prepared import normalize_quant_state  # the older list form is accepted too (:100-105)

    quant_state = normalize_quant_state(quant_state)
    state2 = quant_state.state2
    if state2 is None or quant_state.absmax.dtype != torch.uint8:
        raise NotImplementedError("only double-quantised NF4 weights (compress_statistics=True) are supported")
    data = W.data if isinstance(W, torch.nn.Parameter) else W
    return fmsa_hip.nf4_dequant(data.reshape(-1), quant_state.absmax, state2.absmax, state2.code, quant_state.code,
                                float(quant_state.offset), tuple(quant_state.shape), quant_state.blocksize,
                                state2.blocksize, out_dtype or quant_state.dtype)
