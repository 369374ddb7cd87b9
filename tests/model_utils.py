"""Builders of small GPTQ + LoRA modules for the module-level tests."""
from __future__ import annotations

import torch
from torch import nn

from oracle import lora as olora
from tests.helpers import make_gptq


class MaskDropout(nn.Module):
    """Deterministic stand-in for nn.Dropout: multiplies by a fixed 0/1 mask, no 1/(1-p) rescale
    (the reference's test double, plugins/fused-ops-and-kernels/tests/test_fused_ops.py:68-83)."""

    def __init__(self, p, shape, seed=0):
        super().__init__()
        gen = torch.Generator().manual_seed(seed)
        self.register_buffer("mask", (torch.rand(shape, generator=gen) >= p).float())

    def forward(self, x):
        return x * self.mask.to(x.dtype).reshape(x.shape)


def make_lora_gptq_linear(K, N, r, alpha, seed, group_size=128, act_order=False, bias=False, device="cpu",
                          lora_dtype=torch.float32, dropout=None, order_seed=None):
    """LoraLinear(QuantLinear) with seeded weights.  Returns (module, dense fp32 W [K, N], A, B)."""
    from fms_acceleration_peft import LoraLinear, QuantLinear

    w = make_gptq(K, N, group_size, seed=seed, act_order=bool(act_order), order_seed=order_seed)
    ql = QuantLinear(4, w["group_size"], K, N, bias)
    ql.load_packed(w["np"]["qweight"], w["np"]["qzeros"], w["np"]["scales"], w["np"]["g_idx"])
    if bias:
        gen = torch.Generator().manual_seed(seed + 77)
        ql.bias.copy_((torch.randn(N, generator=gen) * 0.1).half())
    lin = LoraLinear(ql, r, alpha, dtype=lora_dtype)
    A, B = olora.make_lora(K, N, r, seed + 1)
    lin.lora_A["default"].weight.data.copy_(A)
    lin.lora_B["default"].weight.data.copy_(B)
    if dropout is not None:
        lin.lora_dropout["default"] = dropout
    return lin.to(device), w["dense"], A, B


def make_lora_nf4_linear(K, N, r, alpha, seed, bias=False, device="cpu", lora_dtype=torch.float32, dropout=None,
                         compute_dtype=torch.bfloat16):
    """LoraLinear(Linear4bit) with seeded weights; the NF4 tensors come from the oracle's quantiser.
    Returns (module, dense fp32 W [K, N] from the oracle's dequantisation, A, B)."""
    import numpy as np

    from fms_acceleration_peft import Linear4bit, LoraLinear
    from fms_acceleration_peft.nf4 import Params4bit, QuantState, QuantState2
    from oracle import nf4 as onf4

    rng = np.random.default_rng(seed)
    Wd = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    q = onf4.quantize(Wd)
    base = Linear4bit(K, N, bias, compute_dtype)
    state = QuantState(torch.from_numpy(q["absmax_q"]), (N, K), compute_dtype, q["blocksize"],
                       torch.from_numpy(onf4.NF4.copy()), torch.tensor(float(q["offset"])),
                       QuantState2(torch.from_numpy(q["absmax2"]), torch.from_numpy(q["code2"]), q["blocksize2"]))
    base.weight = Params4bit(torch.from_numpy(q["packed"]), state)
    if bias:
        gen = torch.Generator().manual_seed(seed + 77)
        base.bias.data.copy_((torch.randn(N, generator=gen) * 0.1).to(compute_dtype))
    lin = LoraLinear(base, r, alpha, dtype=lora_dtype)
    A, B = olora.make_lora(K, N, r, seed + 1)
    lin.lora_A["default"].weight.data.copy_(A)
    lin.lora_B["default"].weight.data.copy_(B)
    if dropout is not None:
        lin.lora_dropout["default"] = dropout
    return lin.to(device), onf4.dequant(q, "fp32").t().contiguous(), A, B
