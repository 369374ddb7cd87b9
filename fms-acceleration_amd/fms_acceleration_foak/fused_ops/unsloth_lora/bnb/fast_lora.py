"""Fused LoRA autograd functions over a bitsandbytes NF4 base (drop-in counterparts of
fused_ops/unsloth_lora/bnb/fast_lora.py of the reference: `LoRA_MLP` :21-172, `LoRA_QKV` :223-362,
`LoRA_W` :379-458, entry points :176-188, :365-376, :468-471; same positional arguments, same
gradient tuples).

The reference materialises the dense weight (two calls into libbitsandbytes) and contracts it with a
library GEMM.  Here the NF4 codes are re-laid once per (frozen) weight into the word layout of the
fused kernels (fmsa_nf4_prepare) and the same dequant-GEMM kernels as on the GPTQ path read them
directly: the 16-entry code book sits in the lanes of the wave and is gathered per nibble, the product
with the block's absmax is rounded once, and LoRA, bias and SwiGLU are fused into the epilogues.  No
dense copy of the weight is ever written.  Forward / backward bodies are shared with the GPTQ flavour
(fused_core.py).

Departures, as for GPTQ: the down-projection LoRA term of dh is masked by (dropout(h) != 0) instead
of the reference's shape-mismatched in-place mask (:124-127); dX is a fresh tensor (the reference
writes it into the saved X, :152, :337); the activation of the MLP is SwiGLU (the only one the
patch rules bind, models/utils.py:31-42 of the reference), fused into the gate/up epilogue.
"""
from __future__ import annotations

import torch

import fmsa_hip
from fmsa_hip.nf4_prepared import prepare as _prepare

from .. import fused_core as core
from ..fused_core import _act_dtype, _Proj
from ..utils import get_lora_parameters


def _proj(W, W_quant, bias, A, B, S, dtype):
    if W_quant is None:
        raise NotImplementedError("the fused NF4-LoRA ops need a quantised base weight (no quant_state found)")
    return _Proj(_prepare(W, W_quant), bias, A, B, S, dtype)


class LoRA_W(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, X, W, W_quant, bias, A, B, S, dropout_O=None):
        dtype = _act_dtype(X)
        return core.w_forward(ctx, X, _proj(W, W_quant, bias, A, B, S, dtype), dropout_O, dtype)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dY):
        dX, dA, dB = core.w_backward(ctx, dY)
        return dX, None, None, None, dA, dB, None, None


class LoRA_QKV(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, X,
                QW, QW_quant, Q_bias, QA, QB, QS,
                KW, KW_quant, K_bias, KA, KB, KS,
                VW, VW_quant, V_bias, VA, VB, VS,
                dropout_Q=None, dropout_K=None, dropout_V=None):
        dtype = _act_dtype(X)
        projs = [_proj(QW, QW_quant, Q_bias, QA, QB, QS, dtype), _proj(KW, KW_quant, K_bias, KA, KB, KS, dtype),
                 _proj(VW, VW_quant, V_bias, VA, VB, VS, dtype)]
        return core.qkv_forward(ctx, X, projs, (dropout_Q, dropout_K, dropout_V), dtype)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dQ, dK, dV):
        dX, grads = core.qkv_backward(ctx, dQ, dK, dV)
        n3 = (None,) * 3
        return (dX,
                *n3, grads[0][0], grads[0][1], None,
                *n3, grads[1][0], grads[1][1], None,
                *n3, grads[2][0], grads[2][1], None,
                None, None, None)


class LoRA_QKV_RoPE(torch.autograd.Function):
    """LoRA_QKV whose Q and K leave with the rotary position embedding applied in the epilogue of the projection
    kernel (the NF4 twin of gptq/fast_lora.py's LoRA_QKV_RoPE here; kernels/unsloth/rope_embedding.py:36-65 of the
    reference is the separate pass it replaces)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, X, cos, sin, head_dim,
                QW, QW_quant, Q_bias, QA, QB, QS,
                KW, KW_quant, K_bias, KA, KB, KS,
                VW, VW_quant, V_bias, VA, VB, VS,
                dropout_Q=None, dropout_K=None, dropout_V=None):
        dtype = _act_dtype(X)
        projs = [_proj(QW, QW_quant, Q_bias, QA, QB, QS, dtype), _proj(KW, KW_quant, K_bias, KA, KB, KS, dtype),
                 _proj(VW, VW_quant, V_bias, VA, VB, VS, dtype)]
        return core.qkv_forward(ctx, X, projs, (dropout_Q, dropout_K, dropout_V), dtype, rope=(cos, sin, int(head_dim)))

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dQ, dK, dV):
        dX, grads = core.qkv_backward(ctx, dQ, dK, dV)
        n3 = (None,) * 3
        return (dX, None, None, None,
                *n3, grads[0][0], grads[0][1], None,
                *n3, grads[1][0], grads[1][1], None,
                *n3, grads[2][0], grads[2][1], None,
                None, None, None)


def swiglu_fg_kernel(e, g):
    """h = silu(e) * g (reference: fused_ops/unsloth_lora/swiglu.py:40-47)."""
    return fmsa_hip.swiglu_fwd(e, g)


def swiglu_DWf_DW_dfg_kernel(DW, e, g):
    """In place as the reference (:92-98): returns (h, d_g, d_e) with d_g, d_e overwriting e, g."""
    h = fmsa_hip.swiglu_bwd(DW, e, g)
    return h, e, g


class LoRA_MLP(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, X,
                gateW, gateW_quant, gate_bias, gateA, gateB, gateS,
                upW, upW_quant, up_bias, upA, upB, upS,
                downW, downW_quant, down_bias, downA, downB, downS,
                _forward_function, _backward_function,
                dropout_gate=None, dropout_up=None, dropout_down=None):
        if _forward_function is not swiglu_fg_kernel or _backward_function is not swiglu_DWf_DW_dfg_kernel:
            raise NotImplementedError("the fused NF4 MLP computes SwiGLU in its GEMM epilogues; other activations are not built")
        dtype = _act_dtype(X)
        gate = _proj(gateW, gateW_quant, gate_bias, gateA, gateB, gateS, dtype)
        up = _proj(upW, upW_quant, up_bias, upA, upB, upS, dtype)
        down = _proj(downW, downW_quant, down_bias, downA, downB, downS, dtype)
        return core.mlp_forward(ctx, X, gate, up, down, (dropout_gate, dropout_up, dropout_down), dtype)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dY):
        dX, (dAg, dBg), (dAu, dBu), (dAd, dBd) = core.mlp_backward(ctx, dY)
        n3 = (None,) * 3
        return (dX,
                *n3, dAg, dBg, None,
                *n3, dAu, dBu, None,
                *n3, dAd, dBd, None,
                None, None, None, None, None)


def apply_lora_mlp_swiglu(self, X):
    gateW, gateW_quant, gate_bias, gateA, gateB, gateS, dropout_gate = get_lora_parameters(self.gate_proj)
    upW, upW_quant, up_bias, upA, upB, upS, dropout_up = get_lora_parameters(self.up_proj)
    downW, downW_quant, down_bias, downA, downB, downS, dropout_down = get_lora_parameters(self.down_proj)
    return LoRA_MLP.apply(X,
                          gateW, gateW_quant, gate_bias, gateA, gateB, gateS,
                          upW, upW_quant, up_bias, upA, upB, upS,
                          downW, downW_quant, down_bias, downA, downB, downS,
                          swiglu_fg_kernel, swiglu_DWf_DW_dfg_kernel,
                          dropout_gate, dropout_up, dropout_down)


def apply_lora_qkv(self, X):
    QW, QW_quant, Q_bias, QA, QB, QS, dropoutQ = get_lora_parameters(self.q_proj)
    KW, KW_quant, K_bias, KA, KB, KS, dropoutK = get_lora_parameters(self.k_proj)
    VW, VW_quant, V_bias, VA, VB, VS, dropoutV = get_lora_parameters(self.v_proj)
    return LoRA_QKV.apply(X,
                          QW, QW_quant, Q_bias, QA, QB, QS,
                          KW, KW_quant, K_bias, KA, KB, KS,
                          VW, VW_quant, V_bias, VA, VB, VS,
                          dropoutQ, dropoutK, dropoutV)


def apply_lora_qkv_rope(self, X, cos, sin):
    """apply_lora_qkv with the rotary embedding of Q and K fused into the projection launch (see the GPTQ twin)."""
    from ..gptq.fast_lora import rope_tables

    QW, QW_quant, Q_bias, QA, QB, QS, dropoutQ = get_lora_parameters(self.q_proj)
    KW, KW_quant, K_bias, KA, KB, KS, dropoutK = get_lora_parameters(self.k_proj)
    VW, VW_quant, V_bias, VA, VB, VS, dropoutV = get_lora_parameters(self.v_proj)
    batch, seq_len = (X.shape[0], X.shape[1]) if X.dim() == 3 else (1, X.shape[0])
    cos2d, sin2d = rope_tables(cos, sin, batch, seq_len)
    head_dim = getattr(self, "head_dim", None) or self.config.head_dim
    return LoRA_QKV_RoPE.apply(X, cos2d, sin2d, head_dim,
                               QW, QW_quant, Q_bias, QA, QB, QS,
                               KW, KW_quant, K_bias, KA, KB, KS,
                               VW, VW_quant, V_bias, VA, VB, VS,
                               dropoutQ, dropoutK, dropoutV)


def apply_lora_o(self, X):
    OW, OW_quant, O_bias, OA, OB, OS, dropout = get_lora_parameters(self.o_proj)
    return LoRA_W.apply(X, OW, OW_quant, O_bias, OA, OB, OS, dropout)


def apply_lora_o_v2(self, X):
    OW, OW_quant, O_bias, OA, OB, OS, dropout = get_lora_parameters(self)
    return LoRA_W.apply(X, OW, OW_quant, O_bias, OA, OB, OS, dropout)
