"""Seeded synthetic inputs shared by the CPU and GPU tests (weights ~N(0, 0.02) RTN-quantised
to asymmetric 4-bit per group, activations and upstream grads ~N(0, 1))."""
from __future__ import annotations

import numpy as np
import torch

from oracle import gptq as ogptq


def make_gptq(K, N, group_size=128, seed=0, act_order=False, sym=False, v1=False, order_seed=None):
    """Returns dict with numpy QuantLinear buffers, torch CPU tensors, and the fp32 dense weight.
    `order_seed` fixes the act-order permutation independently of the weights, so that several
    projections can share one (as projections quantised on the same input do)."""
    gen = torch.Generator().manual_seed(seed)
    W = (torch.randn(N, K, generator=gen) * 0.02).numpy()
    g_idx = ogptq.act_order_g_idx(K, group_size, seed=seed + 4 if order_seed is None else order_seed) if act_order else None
    buf = ogptq.quantize_and_pack(W, group_size, sym=sym, g_idx=g_idx)
    zero_offset = 0
    if v1:
        buf["qzeros"] = ogptq.to_v1_zeros(buf["qzeros"])
        zero_offset = 1
    dense = ogptq.dequant(buf["qweight"], buf["scales"], buf["qzeros"], buf["g_idx"], zero_offset=zero_offset, out="fp32")
    t = {
        "qweight": torch.from_numpy(buf["qweight"].copy()),
        "qzeros": torch.from_numpy(buf["qzeros"].copy()),
        "scales": torch.from_numpy(buf["scales"].copy()),
        "g_idx": torch.from_numpy(buf["g_idx"].copy()),
    }
    return {"np": buf, "t": t, "dense": dense, "K": K, "N": N, "group_size": buf["group_size"],
            "zero_offset": zero_offset, "act_order": act_order}


def randn(shape, seed, dtype=torch.float32, scale=1.0):
    gen = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)
