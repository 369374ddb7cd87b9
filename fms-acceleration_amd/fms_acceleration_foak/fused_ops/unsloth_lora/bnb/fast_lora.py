"""Fused LoRA autograd functions over a bitsandbytes NF4 base (drop-in counterparts of
fused_ops/unsloth_lora/bnb/fast_lora.py of the reference: `LoRA_MLP` :21-172, `LoRA_QKV` :223-362,
`LoRA_W` :379-458, entry points :176-188, :365-376, :468-471; same positional arguments, same
gradient tuples).

Structure of this NF4 path: the base weight is materialised by libfmsa_hip's one-pass NF4 kernel
(the reference makes two calls into libbitsandbytes) and contracted with a plain library GEMM, as the
reference does; everything LoRA- and SwiGLU-specific runs on the hand-written kernels shared with
the GPTQ path: `fmsa_lora_down` (Xd A^T, dY B), `fmsa_lora_grad` (deterministic dA, dB) and the
SwiGLU forward / in-place backward.  A fused NF4 operand loader for the MFMA GEMMs (as the GPTQ path
has) is not built.

Departures, as for GPTQ: the down-projection LoRA term of dh is masked by (dropout(h) != 0) instead
of the reference's shape-mismatched in-place mask (:124-127); dX is a fresh tensor (the reference
writes it into the saved X, :152, :337).
"""
from __future__ import annotations

import torch

import fmsa_hip

from ..utils import fast_dequantize, get_lora_parameters


def _act_dtype(X):
    if X.dtype in (torch.float16, torch.bfloat16):
        return X.dtype
    if torch.is_autocast_enabled():
        return torch.get_autocast_gpu_dtype()
    raise TypeError(f"fused NF4-LoRA ops compute in float16 / bfloat16, got {X.dtype} outside autocast")


def _as2d(X, dtype):
    X2 = X.reshape(-1, X.shape[-1])
    if X2.dtype != dtype:
        X2 = X2.to(dtype)
    return X2 if X2.is_contiguous() else X2.contiguous()


def _apply_dropout(X2, dropout):
    if dropout is None or isinstance(dropout, torch.nn.Identity):
        return X2
    if isinstance(dropout, torch.Tensor):
        return X2 * dropout.reshape(X2.shape).to(X2.dtype)
    Xd = dropout(X2)
    return Xd if Xd.is_contiguous() else Xd.contiguous()


class _Proj:
    def __init__(self, W, W_quant, bias, A, B, S, dtype):
        self.W, self.W_quant = W, W_quant
        self.bias = None if bias is None else bias.to(dtype)
        self.A_param, self.B_param = A, B
        self.r = 0 if A is None else A.shape[0]
        self.s = 0.0 if S is None else float(S)
        self.A = self.At = self.B = self.Bt = None  # [r, K], [K, r], [N, r], [r, N] in the activation dtype
        if A is not None:
            self.A, self.At, self.B, self.Bt = fmsa_hip.lora_pack(A, B, dtype)
        self.dtype = dtype

    def dense(self):
        """[N, K] in the activation dtype (one rounding of code * absmax)."""
        return fast_dequantize(self.W, self.W_quant, self.dtype)

    def forward(self, X2, Xd):
        """Y = X W^T + s (Xd A^T) B^T (+ bias); returns (Y, U)."""
        Y = X2 @ self.dense().t()
        U = None
        if self.r:
            U = fmsa_hip.lora_down(Xd, self.A)
            Y.addmm_(U, self.Bt, alpha=self.s)
        if self.bias is not None:
            Y += self.bias
        return Y, U

    def dx(self, dY2, T, Xd):
        """dY W + (Xd != 0) * s (T A)."""
        dX = dY2 @ self.dense()
        if self.r:
            lora = (T @ self.A) * self.s
            dX += lora * (Xd != 0) if Xd is not None else lora
        return dX

    def lora_grads(self, T, Xd, U, dY2):
        if not self.r:
            return None, None
        dA = fmsa_hip.lora_grad(T, Xd, self.s, False, self.A_param.dtype)
        dB = fmsa_hip.lora_grad(U, dY2, self.s, True, self.B_param.dtype)
        return dA, dB

    def T(self, dY2):
        return fmsa_hip.lora_down(dY2, self.Bt) if self.r else None


class LoRA_W(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, X, W, W_quant, bias, A, B, S, dropout_O=None):
        dtype = _act_dtype(X)
        X2 = _as2d(X, dtype)
        p = _Proj(W, W_quant, bias, A, B, S, dtype)
        Xd = _apply_dropout(X2, dropout_O) if p.r else X2
        Y, U = p.forward(X2, Xd)
        ctx.proj, ctx.act_dtype, ctx.x_shape, ctx.x_dtype = p, dtype, X.shape, X.dtype
        ctx.save_for_backward(Xd, U) if p.r else ctx.save_for_backward()
        return Y.view(*X.shape[:-1], Y.shape[-1])

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dY):
        p = ctx.proj
        dY2 = _as2d(dY, ctx.act_dtype)
        T = Xd = U = None
        if p.r:
            Xd, U = ctx.saved_tensors
            T = p.T(dY2)
        dA, dB = p.lora_grads(T, Xd, U, dY2)
        dX = p.dx(dY2, T, Xd)
        return dX.view(ctx.x_shape).to(ctx.x_dtype), None, None, None, dA, dB, None, None


class LoRA_QKV(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, X,
                QW, QW_quant, Q_bias, QA, QB, QS,
                KW, KW_quant, K_bias, KA, KB, KS,
                VW, VW_quant, V_bias, VA, VB, VS,
                dropout_Q=None, dropout_K=None, dropout_V=None):
        dtype = _act_dtype(X)
        X2 = _as2d(X, dtype)
        projs = [_Proj(QW, QW_quant, Q_bias, QA, QB, QS, dtype), _Proj(KW, KW_quant, K_bias, KA, KB, KS, dtype),
                 _Proj(VW, VW_quant, V_bias, VA, VB, VS, dtype)]
        outs, saved, layout = [], [], []
        for p, d in zip(projs, (dropout_Q, dropout_K, dropout_V)):
            Xd = _apply_dropout(X2, d) if p.r else X2
            Y, U = p.forward(X2, Xd)
            outs.append(Y.view(*X.shape[:-1], Y.shape[-1]))
            layout.append(bool(p.r))
            if p.r:
                saved += [Xd, U]
        ctx.projs, ctx.layout, ctx.act_dtype, ctx.x_shape, ctx.x_dtype = projs, layout, dtype, X.shape, X.dtype
        ctx.save_for_backward(*saved)
        return tuple(outs)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dQ, dK, dV):
        saved = list(ctx.saved_tensors)
        dX, grads = None, []
        for p, dY, has in zip(ctx.projs, (dQ, dK, dV), ctx.layout):
            dY2 = _as2d(dY, ctx.act_dtype)
            T = Xd = U = None
            if has:
                Xd, U = saved.pop(0), saved.pop(0)
                T = p.T(dY2)
            grads.append(p.lora_grads(T, Xd, U, dY2))
            part = p.dx(dY2, T, Xd)
            dX = part if dX is None else dX.add_(part)
        n3 = (None,) * 3
        return (dX.view(ctx.x_shape).to(ctx.x_dtype),
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
        dtype = _act_dtype(X)
        X2 = _as2d(X, dtype)
        gate = _Proj(gateW, gateW_quant, gate_bias, gateA, gateB, gateS, dtype)
        up = _Proj(upW, upW_quant, up_bias, upA, upB, upS, dtype)
        down = _Proj(downW, downW_quant, down_bias, downA, downB, downS, dtype)
        Xg = _apply_dropout(X2, dropout_gate) if gate.r else X2
        Xu = _apply_dropout(X2, dropout_up) if up.r else X2
        e, Ug = gate.forward(X2, Xg)
        g, Uu = up.forward(X2, Xu)
        h = _forward_function(e, g)
        hd = _apply_dropout(h, dropout_down) if down.r else h
        out, Ud = down.forward(h, hd)
        ctx.projs, ctx.bwd_fn = (gate, up, down), _backward_function
        ctx.act_dtype, ctx.x_shape, ctx.x_dtype = dtype, X.shape, X.dtype
        ctx.down_dropped = hd is not h
        none = X2.new_empty(0)
        ctx.save_for_backward(Xg, Xu, e, g, hd if ctx.down_dropped else none,
                              Ug if gate.r else none, Uu if up.r else none, Ud if down.r else none)
        return out.view(*X.shape[:-1], out.shape[-1])

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dY):
        gate, up, down = ctx.projs
        Xg, Xu, e, g, hd, Ug, Uu, Ud = ctx.saved_tensors
        dY2 = _as2d(dY, ctx.act_dtype)
        Td = down.T(dY2)
        # dh = dY W_d + mask (.) s (T_d A_d); the mask needs h = silu(e) * g before e, g are overwritten
        h_for_mask = hd if ctx.down_dropped else swiglu_fg_kernel(e, g)
        dh = down.dx(dY2, Td, h_for_mask if down.r else None)
        h, d_g, d_e = ctx.bwd_fn(dh, e, g)
        dAd = dBd = None
        if down.r:
            Ud_b = fmsa_hip.lora_down(h, down.A) if ctx.down_dropped else Ud
            dAd, dBd = down.lora_grads(Td, h, Ud_b, dY2)
        Tu, Tg = up.T(d_g), gate.T(d_e)
        dAu, dBu = up.lora_grads(Tu, Xu, Uu, d_g)
        dAg, dBg = gate.lora_grads(Tg, Xg, Ug, d_e)
        dX = up.dx(d_g, Tu, Xu)
        dX += gate.dx(d_e, Tg, Xg)
        n3 = (None,) * 3
        return (dX.view(ctx.x_shape).to(ctx.x_dtype),
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


def apply_lora_o(self, X):
    OW, OW_quant, O_bias, OA, OB, OS, dropout = get_lora_parameters(self.o_proj)
    return LoRA_W.apply(X, OW, OW_quant, O_bias, OA, OB, OS, dropout)


def apply_lora_o_v2(self, X):
    OW, OW_quant, O_bias, OA, OB, OS, dropout = get_lora_parameters(self)
    return LoRA_W.apply(X, OW, OW_quant, O_bias, OA, OB, OS, dropout)
