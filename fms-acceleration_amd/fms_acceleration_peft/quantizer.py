"""Round-to-nearest GPTQ-format quantiser, vectorised in torch (CPU or GPU).

Restates the min/max `Quantizer` of the reference (gptqmodel/quantization/quantizer.py:14-18 and
:49-90: per output row and per group, xmin = min(min, 0), xmax = max(max, 0), (0, 0) -> (-1, 1),
scale = (xmax - xmin) / maxq, zero = round(-xmin / scale), q = clamp(round(w / scale) + zero, 0, maxq))
and the packing of QuantLinear.pack (nn_modules/qlinear/qlinear_tritonv2.py:104-165).  It produces
the buffers of a QuantLinear from a dense weight; it is how synthetic checkpoints are made for the
tests and the benchmark (the reference's Hessian-based GPTQ solver is an offline tool and is not
part of the fused-LoRA path).
"""
from __future__ import annotations

import torch


def _pack_dim(vals: torch.Tensor, dim: int, bits: int = 4) -> torch.Tensor:
    """Pack groups of 32/bits consecutive entries along `dim` into int32 words, first entry in the
    low bits."""
    pf = 32 // bits
    v = vals.to(torch.int64).movedim(dim, -1)
    v = v.reshape(*v.shape[:-1], v.shape[-1] // pf, pf)
    shifts = torch.arange(pf, device=v.device, dtype=torch.int64) * bits
    words = (v << shifts).sum(dim=-1)  # < 2**32
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32)
    return words.movedim(-1, dim).contiguous()


@torch.no_grad()
def rtn_quantize(W: torch.Tensor, bits: int = 4, group_size: int = 128, sym: bool = False, g_idx: torch.Tensor = None):
    """W [N, K] (nn.Linear layout) -> dict(qweight int32 [K/8, N], qzeros int32 [G, N/8],
    scales fp16 [G, N], g_idx int32 [K], group_size).  With `g_idx` (act-order) group g consists of
    the columns k with g_idx[k] == g; every group must have exactly group_size members."""
    assert bits == 4
    W = W.float()
    N, K = W.shape
    if group_size == -1:
        group_size = K
    assert K % group_size == 0
    G = K // group_size
    maxq = 2 ** bits - 1
    if g_idx is None:
        g_idx = (torch.arange(K, device=W.device) // group_size).to(torch.int32)
        order = torch.arange(K, device=W.device)
    else:
        g_idx = g_idx.to(W.device).to(torch.int32)
        order = torch.argsort(g_idx.long(), stable=True)  # columns sorted by group
    Ws = W[:, order].reshape(N, G, group_size)
    zero_t = torch.zeros((), device=W.device)
    xmin = torch.minimum(Ws.amin(dim=2), zero_t)
    xmax = torch.maximum(Ws.amax(dim=2), zero_t)
    if sym:
        xmax = torch.maximum(xmin.abs(), xmax)
        xmin = torch.where(xmin < 0, -xmax, xmin)
    dead = (xmin == 0) & (xmax == 0)
    xmin = torch.where(dead, torch.full_like(xmin, -1.0), xmin)
    xmax = torch.where(dead, torch.full_like(xmax, 1.0), xmax)
    scale = (xmax - xmin) / maxq  # [N, G] fp32
    zero = torch.full_like(scale, (maxq + 1) / 2) if sym else torch.round(-xmin / scale)
    q_sorted = torch.clamp(torch.round(Ws / scale[:, :, None]) + zero[:, :, None], 0, maxq)  # [N, G, gs]
    q = torch.empty((N, K), device=W.device, dtype=torch.int64)
    q[:, order] = q_sorted.reshape(N, K).to(torch.int64)
    return {
        "qweight": _pack_dim(q.t().contiguous(), 0),          # [K/8, N]
        "qzeros": _pack_dim(zero.t().contiguous().to(torch.int64), 1),  # [G, N/8]
        "scales": scale.t().contiguous().to(torch.float16),   # [G, N]
        "g_idx": g_idx.contiguous(),
        "group_size": group_size,
    }


def quantize_linear(weight: torch.Tensor, group_size: int = 128, g_idx: torch.Tensor = None, bias: torch.Tensor = None):
    """A QuantLinear holding the RTN quantisation of `weight` [N, K]."""
    from .qlinear import QuantLinear

    N, K = weight.shape
    buf = rtn_quantize(weight, 4, group_size, g_idx=g_idx)
    ql = QuantLinear(4, buf["group_size"], K, N, bias is not None)
    ql.load_packed(buf["qweight"], buf["qzeros"], buf["scales"], buf["g_idx"], bias)
    return ql
