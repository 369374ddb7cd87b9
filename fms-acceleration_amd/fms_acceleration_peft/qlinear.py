"""QuantLinear: the on-device GPTQ data layout, and the UNFUSED forward/backward on the HIP kernels.

Buffer names, shapes and dtypes are those of the reference's tritonv2 QuantLinear
(gptqmodel/nn_modules/qlinear/qlinear_tritonv2.py:67-99), so a state_dict of one loads into the
other.  `forward` is the module-level path without LoRA fusion (`QuantLinearFunction`,
gptqmodel/nn_modules/triton_utils/dequant.py:132-161: base projection only, no gradient for the
frozen weight): what a PEFT LoRA layer calls when the fused-LoRA rules are not installed.
"""
from __future__ import annotations

import math

import numpy as np
import torch
from torch import nn


class QuantLinearFunction(torch.autograd.Function):
    """y = x @ deq(W); dx = dy @ deq(W)^T (dequant.py:141-161).

    bf16 / fp16 activations go through the fused dequant-GEMM kernels with the adapter disabled
    (r = 0): the 4-bit weight is unpacked in registers on its way into the MFMA and no dense matrix
    is ever written.  Other activation types (fp32) take the dequantise-then-matmul route, with the
    dense weight produced in the activation dtype by one rounding."""

    @staticmethod
    def forward(ctx, x, qweight, scales, qzeros, g_idx, bits, group_size, zero_offset):
        import fmsa_hip

        if bits != 4:
            raise NotImplementedError("the gfx950 kernels cover 4-bit GPTQ only")
        ctx.save_for_backward(qweight, scales, qzeros, g_idx)
        ctx.meta = (bits, group_size, zero_offset)
        ctx.fused = x.dtype in (torch.float16, torch.bfloat16) and group_size % 16 == 0
        if not ctx.fused:
            W = fmsa_hip.gptq_dequant(qweight, scales, qzeros, g_idx, group_size, zero_offset, x.dtype)
            return x @ W
        from fmsa_hip.gptq_prepared import prepare

        w = prepare(qweight, scales, qzeros, g_idx, bits)
        x2 = x if x.is_contiguous() else x.contiguous()
        if w.perm is not None:  # act-order: the repacked weight walks K in sorted-group order
            x2 = fmsa_hip.permute_cols(x2, w.perm, gather=True)
        struct = w.struct_interleaved if w.interleaved_ok(x2.dtype) else w.struct
        (y,) = fmsa_hip.gptq_lora_fwd(x2, [{"w": struct, "U": None, "B": None, "bias": None, "r": 0, "s": 0.0}])
        return y

    @staticmethod
    def backward(ctx, dy):
        import fmsa_hip

        qweight, scales, qzeros, g_idx = ctx.saved_tensors
        bits, group_size, zero_offset = ctx.meta
        if not ctx.fused or group_size < 32:
            W = fmsa_hip.gptq_dequant(qweight, scales, qzeros, g_idx, group_size, zero_offset, dy.dtype)
            return dy @ W.t(), None, None, None, None, None, None, None
        from fmsa_hip.gptq_prepared import prepare

        w = prepare(qweight, scales, qzeros, g_idx, bits)
        dy2 = dy if dy.is_contiguous() else dy.contiguous()
        dx = fmsa_hip.gptq_lora_bwd_dx(
            [{"w": w.struct, "nsz": w.nsz, "dY": dy2, "T": None, "At": None, "mask_src": None, "r": 0, "s": 0.0,
              "qweight_t": w.twin[0], "scale_f32": w.twin[1], "negzp_f16": w.twin[2]}], dy2.shape[0], w.K)
        if w.perm is not None:
            dx = fmsa_hip.permute_cols(dx, w.perm, gather=False)
        return dx, None, None, None, None, None, None, None


class QuantLinear(nn.Module):
    QUANT_TYPE = "tritonv2"

    def __init__(self, bits, group_size, infeatures, outfeatures, bias, **kwargs):
        super().__init__()
        if bits not in [2, 4, 8]:
            raise NotImplementedError("Only 2,4,8 bits are supported.")
        if infeatures % 32 != 0 or outfeatures % 32 != 0:
            raise NotImplementedError("in_feature and out_feature must be divisible by 32.")
        self.infeatures = infeatures
        self.outfeatures = outfeatures
        self.bits = bits
        self.group_size = group_size if group_size != -1 else infeatures
        self.maxq = 2 ** self.bits - 1
        n_groups = math.ceil(infeatures / self.group_size)
        self.register_buffer("qweight", torch.zeros((infeatures // 32 * bits, outfeatures), dtype=torch.int32))
        self.register_buffer("qzeros", torch.zeros((n_groups, outfeatures // 32 * bits), dtype=torch.int32))
        self.register_buffer("scales", torch.zeros((n_groups, outfeatures), dtype=torch.float16))
        self.register_buffer("g_idx", (torch.arange(infeatures) // self.group_size).to(torch.int32))
        if bias:
            self.register_buffer("bias", torch.zeros((outfeatures,), dtype=torch.float16))
        else:
            self.bias = None

    def post_init(self):
        pass

    # convenience used by tests / benches: adopt already packed buffers (numpy or torch)
    def load_packed(self, qweight, qzeros, scales, g_idx=None, bias=None):
        def t(x, dt):
            x = torch.from_numpy(np.ascontiguousarray(x)) if isinstance(x, np.ndarray) else x
            return x.to(dt)

        self.qweight.copy_(t(qweight, torch.int32))
        self.qzeros.copy_(t(qzeros, torch.int32))
        self.scales.copy_(t(scales, torch.float16))
        if g_idx is not None:
            self.g_idx.copy_(t(g_idx, torch.int32))
        if bias is not None:
            self.bias.copy_(t(bias, torch.float16))
        return self

    def pack(self, linear, scales, zeros, g_idx=None):
        """Pack an nn.Linear given per-group scales/zeros [N, G] (qlinear_tritonv2.py:104-165)."""
        W = linear.weight.data.clone().float()  # [N, K]
        if g_idx is not None:
            self.g_idx = g_idx.clone().to(torch.int32)
        scales = scales.t().contiguous().float()  # [G, N]
        zeros = zeros.t().contiguous().float()
        self.scales = scales.clone().half()
        if linear.bias is not None:
            self.bias = linear.bias.clone().half()
        g = self.g_idx.long()
        q = torch.round((W.t() + (zeros * scales)[g]) / self.scales.float()[g]).to(torch.int64)  # [K, N]
        pf = 32 // self.bits
        qn = q.numpy().astype(np.uint32)  # [K, N]
        qw = np.zeros((qn.shape[0] // pf, qn.shape[1]), dtype=np.uint32)
        for j in range(pf):  # row pf*i + j -> bits [bits*j, bits*(j+1)) of word i
            qw |= qn[j::pf, :] << np.uint32(self.bits * j)
        self.qweight = torch.from_numpy(qw.view(np.int32))
        zn = zeros.numpy().astype(np.uint32)  # [G, N]
        qz = np.zeros((zn.shape[0], zn.shape[1] // pf), dtype=np.uint32)
        for j in range(pf):  # column pf*i + j -> bits [bits*j, bits*(j+1)) of word i
            qz |= zn[:, j::pf] << np.uint32(self.bits * j)
        self.qzeros = torch.from_numpy(qz.view(np.int32))

    def forward(self, x):
        out_shape = x.shape[:-1] + (self.outfeatures,)
        zero_offset = int(getattr(self.qzeros, "offset", 0) or 0)
        out = QuantLinearFunction.apply(
            x.reshape(-1, x.shape[-1]), self.qweight, self.scales, self.qzeros, self.g_idx, self.bits,
            self.group_size, zero_offset,
        )
        out = out.reshape(out_shape)
        return out + self.bias.to(out.dtype) if self.bias is not None else out
