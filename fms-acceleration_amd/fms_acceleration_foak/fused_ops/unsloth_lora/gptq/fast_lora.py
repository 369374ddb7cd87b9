"""Fused GPTQ-LoRA autograd functions on the gfx950 kernels of libfmsa_hip.

Drop-in counterparts of the reference's `LoRA_MLP`, `LoRA_QKV`, `LoRA_W` and their module-level
entry points (fused_ops/unsloth_lora/gptq/fast_lora.py: :174-435, :466-711, :742-846, entry points
:438-463, :714-739, :849-859): same names, same positional argument order per projection
(`qweight, scales, qzeros, g_idx, bits, bias, A, B, S`), same gradient tuple (None for every frozen
or non-tensor input, dA / dB in the layouts of `lora_A.weight` [r, K] and `lora_B.weight` [N, r]).

What differs is where the work happens.  The reference dequantises W to a dense fp16 matrix and
calls torch.matmul plus ~20 small GEMMs and elementwise kernels per function; here each function
is a handful of launches:

  forward   U = Xd A^T                 (fmsa_lora_down, streams X once)
            Y = X deq(W) + s U B^T     (fmsa_gptq_lora_fwd: nibble unpack in registers -> MFMA,
                                        LoRA / bias / SwiGLU in the epilogue)
  backward  T = dY B                   (fmsa_lora_down)
            dA = s T^T Xd, dB = s dY^T U   (fmsa_lora_grad, deterministic)
            dX = dY deq(W)^T + (Xd != 0) * T (s A)      (fmsa_gptq_lora_bwd_dx)

There is no CPU or PyTorch fallback: tensors must live on the GPU and the library must be built.

Known, documented departures from the reference text:
  * LoRA_MLP.backward masks the LoRA part of dh with (dropout(h) != 0), the form the reference
    uses for every other projection; its own line (:354-357) multiplies dY in place by a mask of
    h's shape and cannot run when hidden != intermediate.
  * Like the reference (UL/swiglu.py:86-88) the MLP backward overwrites the saved e and g, so a
    graph can be back-propagated once (no retain_graph / double backward).
  * 4-bit only (the reference's dequant also accepts 2 and 8 bits).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from fmsa_hip.gptq_prepared import prepare as _prepare  # per-weight C-ABI view, cached on the qweight tensor

from .. import fused_core as core
from ..fused_core import _act_dtype, _Proj


# ----------------------------------------------------------------------------------------------
# quantisation state (mirrors GPTQuantState / extract_gptq_state / get_lora_parameters, :19-116)
# ----------------------------------------------------------------------------------------------
@dataclass
class GPTQuantState:
    infeatures: int
    outfeatures: int
    bits: int
    group_size: int
    maxq: int
    qweight: torch.Tensor
    qzeros: torch.Tensor
    scales: torch.Tensor
    g_idx: torch.Tensor
    bias: Optional[torch.Tensor] = None


def unpack_gptqstate(qstate):
    return qstate.qweight, qstate.scales, qstate.qzeros, qstate.g_idx, qstate.bits


def _nonzero_bias(qmodule):
    """The reference drops an all-zero bias (:63-67) with a count_nonzero per call; the answer is
    cached on the tensor and refreshed when the tensor is modified."""
    bias = getattr(qmodule, "bias", None)
    if bias is None:
        return None
    cached = getattr(bias, "_fmsa_nonzero", None)
    if cached is None or cached[0] != bias._version:
        cached = (bias._version, bool(bias.count_nonzero() > 0))
        bias._fmsa_nonzero = cached
    return bias if cached[1] else None


def extract_gptq_state(qmodule):
    if hasattr(qmodule, "base_layer"):
        qmodule = qmodule.base_layer
    return GPTQuantState(
        infeatures=qmodule.infeatures,
        outfeatures=qmodule.outfeatures,
        bits=qmodule.bits,
        group_size=qmodule.group_size,
        maxq=qmodule.maxq,
        qweight=qmodule.qweight,
        qzeros=qmodule.qzeros,
        scales=qmodule.scales,
        g_idx=qmodule.g_idx,
        bias=_nonzero_bias(qmodule),
    )


def get_lora_parameters(proj):
    """(qstate, bias, A, B, s, dropout) of a LoRA-wrapped (or bare) GPTQ linear; A = B = s = None
    when the adapters are disabled or merged (:94-116)."""
    base_layer = proj.base_layer if hasattr(proj, "base_layer") else proj
    qstate = extract_gptq_state(base_layer)
    bias = qstate.bias
    if base_layer.__module__.startswith("auto_gptq"):
        # checkpoints packed by the external auto_gptq library keep zero-1 in qzeros
        setattr(qstate.qzeros, "offset", 1)
    if not hasattr(proj, "disable_adapters") or proj.disable_adapters or proj.merged:
        return qstate, bias, None, None, None, None
    active = proj.active_adapters[0] if hasattr(proj, "active_adapters") else proj.active_adapter
    A = proj.lora_A[active].weight
    B = proj.lora_B[active].weight
    s = proj.scaling[active]
    dropout = proj.lora_dropout[active] if hasattr(proj, "lora_dropout") else None
    return qstate, bias, A, B, s, dropout



def _proj(args, dtype):
    qweight, scales, qzeros, g_idx, bits, bias, A, B, S = args
    return _Proj(_prepare(qweight, scales, qzeros, g_idx, bits), bias, A, B, S, dtype)


# ----------------------------------------------------------------------------------------------
# LoRA_W  (o_proj)
# ----------------------------------------------------------------------------------------------
class LoRA_W(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, X, O_qweight, O_scales, O_qzeros, O_g_idx, O_bits, O_bias, A, B, S, dropout_O=None):
        dtype = _act_dtype(X)
        p = _proj((O_qweight, O_scales, O_qzeros, O_g_idx, O_bits, O_bias, A, B, S), dtype)
        return core.w_forward(ctx, X, p, dropout_O, dtype)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dY):
        dX, dA, dB = core.w_backward(ctx, dY)
        return (dX, None, None, None, None, None, None, dA, dB, None, None)


# ----------------------------------------------------------------------------------------------
# LoRA_QKV
# ----------------------------------------------------------------------------------------------
class LoRA_QKV(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(
        ctx, X,
        Q_qweight, Q_scales, Q_qzeros, Q_g_idx, Q_bits, Q_bias, QA, QB, QS,
        K_qweight, K_scales, K_qzeros, K_g_idx, K_bits, K_bias, KA, KB, KS,
        V_qweight, V_scales, V_qzeros, V_g_idx, V_bits, V_bias, VA, VB, VS,
        dropout_Q=None, dropout_K=None, dropout_V=None,
    ):
        dtype = _act_dtype(X)
        projs = [
            _proj((Q_qweight, Q_scales, Q_qzeros, Q_g_idx, Q_bits, Q_bias, QA, QB, QS), dtype),
            _proj((K_qweight, K_scales, K_qzeros, K_g_idx, K_bits, K_bias, KA, KB, KS), dtype),
            _proj((V_qweight, V_scales, V_qzeros, V_g_idx, V_bits, V_bias, VA, VB, VS), dtype),
        ]
        return core.qkv_forward(ctx, X, projs, (dropout_Q, dropout_K, dropout_V), dtype)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dQ, dK, dV):
        dX, grads = core.qkv_backward(ctx, dQ, dK, dV)
        n6 = (None,) * 6
        return (
            dX,
            *n6, grads[0][0], grads[0][1], None,
            *n6, grads[1][0], grads[1][1], None,
            *n6, grads[2][0], grads[2][1], None,
            None, None, None,
        )


class LoRA_QKV_RoPE(torch.autograd.Function):
    """LoRA_QKV whose Q and K leave with the rotary position embedding applied (the forward kernel rotates in its
    epilogue instead of a separate pass of kernels/unsloth/rope_embedding.py over Q and K); V is untouched.  cos / sin:
    [positions, head_dim] tables (or [batch * seq, head_dim], used row by row); the token at flattened row m takes
    table row m % positions.  The backward rotates dQ and dK back before the LoRA_QKV backward."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(
        ctx, X, cos, sin, head_dim,
        Q_qweight, Q_scales, Q_qzeros, Q_g_idx, Q_bits, Q_bias, QA, QB, QS,
        K_qweight, K_scales, K_qzeros, K_g_idx, K_bits, K_bias, KA, KB, KS,
        V_qweight, V_scales, V_qzeros, V_g_idx, V_bits, V_bias, VA, VB, VS,
        dropout_Q=None, dropout_K=None, dropout_V=None,
    ):
        dtype = _act_dtype(X)
        projs = [
            _proj((Q_qweight, Q_scales, Q_qzeros, Q_g_idx, Q_bits, Q_bias, QA, QB, QS), dtype),
            _proj((K_qweight, K_scales, K_qzeros, K_g_idx, K_bits, K_bias, KA, KB, KS), dtype),
            _proj((V_qweight, V_scales, V_qzeros, V_g_idx, V_bits, V_bias, VA, VB, VS), dtype),
        ]
        return core.qkv_forward(ctx, X, projs, (dropout_Q, dropout_K, dropout_V), dtype, rope=(cos, sin, int(head_dim)))

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dQ, dK, dV):
        dX, grads = core.qkv_backward(ctx, dQ, dK, dV)
        n6 = (None,) * 6
        return (
            dX, None, None, None,
            *n6, grads[0][0], grads[0][1], None,
            *n6, grads[1][0], grads[1][1], None,
            *n6, grads[2][0], grads[2][1], None,
            None, None, None,
        )


# ----------------------------------------------------------------------------------------------
# LoRA_MLP  (SwiGLU)
# ----------------------------------------------------------------------------------------------
class LoRA_MLP(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(
        ctx, X,
        gate_qweight, gate_scales, gate_qzeros, gate_g_idx, gate_bits, gate_bias, gateA, gateB, gateS,
        up_qweight, up_scales, up_qzeros, up_g_idx, up_bits, up_bias, upA, upB, upS,
        down_qweight, down_scales, down_qzeros, down_g_idx, down_bits, down_bias, downA, downB, downS,
        dropout_gate=None, dropout_up=None, dropout_down=None,
    ):
        dtype = _act_dtype(X)
        gate = _proj((gate_qweight, gate_scales, gate_qzeros, gate_g_idx, gate_bits, gate_bias, gateA, gateB, gateS), dtype)
        up = _proj((up_qweight, up_scales, up_qzeros, up_g_idx, up_bits, up_bias, upA, upB, upS), dtype)
        down = _proj((down_qweight, down_scales, down_qzeros, down_g_idx, down_bits, down_bias, downA, downB, downS), dtype)
        return core.mlp_forward(ctx, X, gate, up, down, (dropout_gate, dropout_up, dropout_down), dtype)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dY):
        dX, (dAg, dBg), (dAu, dBu), (dAd, dBd) = core.mlp_backward(ctx, dY)
        n6 = (None,) * 6
        return (
            dX,
            *n6, dAg, dBg, None,
            *n6, dAu, dBu, None,
            *n6, dAd, dBd, None,
            None, None, None,
        )


# ----------------------------------------------------------------------------------------------
# module-level entry points (bound to modules with MethodType by the model patcher)
# ----------------------------------------------------------------------------------------------
def apply_lora_mlp(self, X):
    gateQstate, gate_bias, gateA, gateB, gateS, dropout_gate = get_lora_parameters(self.gate_proj)
    upQState, up_bias, upA, upB, upS, dropout_up = get_lora_parameters(self.up_proj)
    downQState, down_bias, downA, downB, downS, dropout_down = get_lora_parameters(self.down_proj)
    return LoRA_MLP.apply(
        X,
        *unpack_gptqstate(gateQstate), gate_bias, gateA, gateB, gateS,
        *unpack_gptqstate(upQState), up_bias, upA, upB, upS,
        *unpack_gptqstate(downQState), down_bias, downA, downB, downS,
        dropout_gate, dropout_up, dropout_down,
    )


def apply_lora_qkv(self, X):
    Qqstate, Q_bias, QA, QB, QS, Qdropout = get_lora_parameters(self.q_proj)
    Kqstate, K_bias, KA, KB, KS, Kdropout = get_lora_parameters(self.k_proj)
    Vqstate, V_bias, VA, VB, VS, Vdropout = get_lora_parameters(self.v_proj)
    return LoRA_QKV.apply(
        X,
        *unpack_gptqstate(Qqstate), Q_bias, QA, QB, QS,
        *unpack_gptqstate(Kqstate), K_bias, KA, KB, KS,
        *unpack_gptqstate(Vqstate), V_bias, VA, VB, VS,
        Qdropout, Kdropout, Vdropout,
    )


def rope_tables(cos, sin, batch, seq_len):
    """cos / sin as transformers passes them ([1 or batch, seq, head_dim], or a [positions, head_dim] cache) ->
    contiguous-row 2-D tables for the kernels: a shared table is cut to seq_len rows (every batch entry restarts at
    position 0), a per-batch table is flattened to [batch * seq, head_dim]."""
    from ....kernels.unsloth.rope_embedding import _rows

    return _rows(cos, batch, seq_len), _rows(sin, batch, seq_len)


def apply_lora_qkv_rope(self, X, cos, sin):
    """apply_lora_qkv with the rotary embedding of Q and K fused into the projection launch.  X [batch, seq, hidden];
    returns (Q, K, V) as [batch, seq, N]; `self.head_dim` (or config.head_dim) gives the head size."""
    Qqstate, Q_bias, QA, QB, QS, Qdropout = get_lora_parameters(self.q_proj)
    Kqstate, K_bias, KA, KB, KS, Kdropout = get_lora_parameters(self.k_proj)
    Vqstate, V_bias, VA, VB, VS, Vdropout = get_lora_parameters(self.v_proj)
    batch, seq_len = (X.shape[0], X.shape[1]) if X.dim() == 3 else (1, X.shape[0])
    cos2d, sin2d = rope_tables(cos, sin, batch, seq_len)
    head_dim = getattr(self, "head_dim", None) or self.config.head_dim
    return LoRA_QKV_RoPE.apply(
        X, cos2d, sin2d, head_dim,
        *unpack_gptqstate(Qqstate), Q_bias, QA, QB, QS,
        *unpack_gptqstate(Kqstate), K_bias, KA, KB, KS,
        *unpack_gptqstate(Vqstate), V_bias, VA, VB, VS,
        Qdropout, Kdropout, Vdropout,
    )


def apply_lora_o(self, X):
    Oqstate, O_bias, OA, OB, OS, dropout = get_lora_parameters(self.o_proj)
    return LoRA_W.apply(X, *unpack_gptqstate(Oqstate), O_bias, OA, OB, OS, dropout)


def apply_lora_o_v2(self, X):
    """Patched directly on the output linear (`self` is the LoRA layer itself, :856-859)."""
    Oqstate, O_bias, OA, OB, OS, dropout = get_lora_parameters(self)
    return LoRA_W.apply(X, *unpack_gptqstate(Oqstate), O_bias, OA, OB, OS, dropout)
