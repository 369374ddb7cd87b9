"""GPTQ 4-bit layout, RTN quantiser and dequantisation, restated on the CPU with numpy.

Layout (GQ/nn_modules/qlinear/qlinear_tritonv2.py:67-99, pack() :104-165):
  qweight int32 [K/8, N]   nibble j of word [k8, n] = q[8*k8 + j, n]
  qzeros  int32 [G, N/8]   nibble j of word [g, n8] = z[g, 8*n8 + j]
  scales  fp16  [G, N]
  g_idx   int32 [K]        default k // group_size (:88-93)
"""
from __future__ import annotations

import numpy as np

BITS = 4
PF = 32 // BITS  # values per int32
MAXQ = (1 << BITS) - 1


# ----------------------------------------------------------------------------------------------
# packing  (qlinear_tritonv2.py:132-165)
# ----------------------------------------------------------------------------------------------
def pack_rows(q: np.ndarray) -> np.ndarray:
    """q int [K, N] in [0, 15] -> qweight int32 [K/8, N]; row 8*i+j goes to bits 4j..4j+3."""
    q = np.asarray(q)
    K, N = q.shape
    assert K % PF == 0
    u = q.astype(np.uint32).reshape(K // PF, PF, N)
    out = np.zeros((K // PF, N), dtype=np.uint32)
    for j in range(PF):
        out |= u[:, j, :] << np.uint32(BITS * j)
    return out.view(np.int32)


def unpack_rows(qweight: np.ndarray) -> np.ndarray:
    """Inverse of pack_rows (UL/gptq/triton/kernels.py:79-100)."""
    u = np.asarray(qweight).view(np.uint32)
    K8, N = u.shape
    out = np.empty((K8, PF, N), dtype=np.int32)
    for j in range(PF):
        out[:, j, :] = (u >> np.uint32(BITS * j)) & np.uint32(MAXQ)
    return out.reshape(K8 * PF, N)


def pack_cols(z: np.ndarray) -> np.ndarray:
    """z int [G, N] in [0, 15] -> qzeros int32 [G, N/8]; column 8*i+j goes to bits 4j..4j+3."""
    z = np.asarray(z)
    G, N = z.shape
    assert N % PF == 0
    u = z.astype(np.uint32).reshape(G, N // PF, PF)
    out = np.zeros((G, N // PF), dtype=np.uint32)
    for j in range(PF):
        out |= u[:, :, j] << np.uint32(BITS * j)
    return out.view(np.int32)


def unpack_cols(qzeros: np.ndarray) -> np.ndarray:
    """Inverse of pack_cols (UL/gptq/triton/kernels.py:103-110)."""
    u = np.asarray(qzeros).view(np.uint32)
    G, N8 = u.shape
    out = np.empty((G, N8, PF), dtype=np.int32)
    for j in range(PF):
        out[:, :, j] = (u >> np.uint32(BITS * j)) & np.uint32(MAXQ)
    return out.reshape(G, N8 * PF)


# ----------------------------------------------------------------------------------------------
# RTN quantiser  (GQ/quantization/quantizer.py:14-18, 49-90; pack() :116, :121-129)
# ----------------------------------------------------------------------------------------------
def rtn_quantize(W: np.ndarray, group_size: int = 128, sym: bool = False, g_idx: np.ndarray | None = None):
    """Round-to-nearest min/max quantisation of W [N, K] (nn.Linear layout), per output row and
    per group of input columns.

    Returns (q int32 [K, N], scales fp16 [G, N], zeros int32 [G, N], g_idx int32 [K]).
    The members of group g are the columns k with g_idx[k] == g (default k // group_size), as in
    GQ/quantization/gptq.py:184-192 for act-order.
    """
    W = np.asarray(W, dtype=np.float32)
    N, K = W.shape
    if group_size == -1:
        group_size = K
    G = -(-K // group_size)
    if g_idx is None:
        g_idx = (np.arange(K) // group_size).astype(np.int32)
    g_idx = np.asarray(g_idx, dtype=np.int32)
    scales = np.empty((G, N), dtype=np.float32)
    zeros = np.empty((G, N), dtype=np.float32)
    q = np.empty((K, N), dtype=np.int32)
    for g in range(G):
        cols = np.nonzero(g_idx == g)[0]
        x = W[:, cols]  # [N, members]
        xmin = np.minimum(x.min(axis=1), 0.0).astype(np.float32)  # quantizer.py:68-70
        xmax = np.maximum(x.max(axis=1), 0.0).astype(np.float32)
        if sym:  # :72-76
            xmax = np.maximum(np.abs(xmin), xmax)
            neg = xmin < 0
            xmin = np.where(neg, -xmax, xmin)
        dead = (xmin == 0) & (xmax == 0)  # :77-79
        xmin = np.where(dead, np.float32(-1), xmin).astype(np.float32)
        xmax = np.where(dead, np.float32(1), xmax).astype(np.float32)
        scale = ((xmax - xmin) / np.float32(MAXQ)).astype(np.float32)  # :85
        if sym:
            zero = np.full_like(scale, (MAXQ + 1) / 2)  # :86-87
        else:
            zero = np.round(-xmin / scale)  # :89  (half-to-even, as torch.round)
        # quantize(): q = clamp(round(x / scale) + zero, 0, maxq)   (:14-18)
        qq = np.clip(np.round(x / scale[:, None]) + zero[:, None], 0, MAXQ)
        q[cols, :] = qq.T.astype(np.int32)
        scales[g] = scale
        zeros[g] = zero
    return q, scales.astype(np.float16), zeros.astype(np.int32), g_idx


def quantize_and_pack(W: np.ndarray, group_size: int = 128, sym: bool = False, g_idx=None):
    """W [N, K] -> dict of QuantLinear buffers (v2 zero-point format: zeros stored as they are)."""
    q, scales, zeros, g_idx = rtn_quantize(W, group_size, sym, g_idx)
    return {
        "qweight": pack_rows(q),
        "qzeros": pack_cols(zeros),
        "scales": scales,
        "g_idx": g_idx,
        "group_size": group_size if group_size != -1 else W.shape[1],
        "K": W.shape[1],
        "N": W.shape[0],
    }


def to_v1_zeros(qzeros_v2: np.ndarray) -> np.ndarray:
    """AutoGPTQ v1 checkpoints store zero-1 in every nibble; the local loader adds 0x11111111 to
    convert (GQ/utils/model.py:230-231).  This is the inverse, used to build v1 test inputs."""
    return (np.asarray(qzeros_v2).view(np.uint32) - np.uint32(0x11111111)).view(np.int32)


# ----------------------------------------------------------------------------------------------
# dequantisation  (UL/gptq/triton/kernels.py:53-122; dequant_ref :15-40)
# ----------------------------------------------------------------------------------------------
def dequant_f64(qweight, scales, qzeros, g_idx=None, group_size: int | None = None, zero_offset: int = 0):
    """W[k, n] = fp32(scales[g, n]) * (q[k, n] - (z[g, n] + zero_offset)), g = g_idx[k], as an
    exact float64 array [K, N].  The product of an fp16 scale (11 significant bits) and an
    integer in [-16, 15] is exact in fp32, hence also here."""
    q = unpack_rows(qweight)  # [K, N]
    z = unpack_cols(qzeros) + int(zero_offset)  # [G, N]
    K, N = q.shape
    G = z.shape[0]
    if g_idx is None:
        assert group_size is not None
        g_idx = np.arange(K) // group_size
    g = np.asarray(g_idx).astype(np.int64)
    g = np.where(g < 0, g + G, g)  # kernels.py:88-91
    s = np.asarray(scales).astype(np.float64)  # fp16 -> exact
    return s[g, :] * (q - z[g, :]).astype(np.float64)


def dequant(qweight, scales, qzeros, g_idx=None, group_size=None, zero_offset=0, out="fp16"):
    """Dequantised weight rounded once (RNE) to `out` in {"fp16", "bf16", "fp32"}.
    fp16 is what dequant248 stores (kernels.py:136); bf16 is the fused kernels' MFMA operand.
    Returns a torch tensor [K, N]."""
    import torch

    w = torch.from_numpy(dequant_f64(qweight, scales, qzeros, g_idx, group_size, zero_offset))
    w32 = w.to(torch.float32)  # exact
    assert torch.equal(w32.to(torch.float64), w)
    return {"fp16": w32.to(torch.float16), "bf16": w32.to(torch.bfloat16), "fp32": w32}[out]


def act_order_g_idx(K: int, group_size: int, seed: int = 4) -> np.ndarray:
    """A desc_act group assignment: the sorted assignment k // group_size carried through a random
    column permutation, so that every group has exactly group_size members
    (GQ/quantization/gptq.py:184-192: g_idx[perm[i]] = i // group_size)."""
    rng = np.random.default_rng(seed)
    perm = rng.permutation(K)
    g = np.empty(K, dtype=np.int32)
    g[perm] = (np.arange(K) // group_size).astype(np.int32)
    return g


def dequant_torch(qweight, scales, qzeros, g_idx, zero_offset: int = 0):
    """The reference's pure-torch `dequant_ref` (UL/gptq/triton/kernels.py:15-40) restated: shift /
    mask unpack of qzeros and qweight, then scales[g_idx] * (q - zeros[g_idx]).  `dequant_ref` adds 1
    to the zeros unconditionally (v1 checkpoints); here that is `zero_offset`.  Returns fp32 [K, N].
    Multi-threaded through torch: this is the dequant step of the CPU baseline."""
    import torch

    qweight, scales, qzeros, g_idx = (torch.as_tensor(t) for t in (qweight, scales, qzeros, g_idx))
    wf = torch.arange(0, 32, BITS, dtype=torch.int32)
    zeros = torch.bitwise_and(torch.bitwise_right_shift(qzeros.unsqueeze(2).expand(-1, -1, PF), wf.view(1, 1, -1)), MAXQ)
    zeros = (zeros + zero_offset).reshape(scales.shape)
    weights = torch.bitwise_and(torch.bitwise_right_shift(qweight.unsqueeze(1).expand(-1, PF, -1), wf.view(1, -1, 1)), MAXQ)
    weights = weights.reshape(-1, weights.shape[2])
    g = g_idx.long()
    return scales.float()[g] * (weights - zeros[g]).float()
