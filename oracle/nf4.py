"""bitsandbytes NF4 (blocksize 64) with 8-bit double-quantised absmax (blocksize 256), on the CPU.

PARITY UNPINNED against bitsandbytes itself: the library (`bitsandbytes`, >=0.45.1 in
plugins/accelerated-peft/requirements.txt:10 of the reference) is absent here and nothing in the
reference tree holds its tables or outputs.  What is restated:
  * the 16-entry NF4 code book (published with QLoRA / in bitsandbytes' functional.py) and the
    storage order -- two codes per byte, the even element in the HIGH nibble;
  * the two-step dequantisation the reference performs (UL/utils.py:114-136):
        absmax[b] = code2[absmax_q[b]] * absmax2[b // 256] + offset        (fp32)
        W[i]      = NF4[nibble(i)] * absmax[i // 64]                        (fp32, then one RNE to dtype)
    over the row-major [N, K] weight, returned transposed as [K, N] (:139-140);
  * the published construction of the signed 8-bit dynamic map used for the absmax (an INPUT of the
    dequantisation -- quant_state.state2.code -- so the kernels are agnostic to its contents).
Pinned here by closed forms and round trips only (tests/test_oracle_nf4.py).
"""
from __future__ import annotations

import numpy as np

NF4 = np.array(
    [-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
     -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
     0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
     0.7229568362236023, 1.0], dtype=np.float32)


def dynamic_map_8bit() -> np.ndarray:
    """Signed dynamic 8-bit map (256 sorted fp32 values in [-1, 1]): for exponent i = 0..6 the
    midpoints of 2**i + 1 boundaries linspace(0.1, 1) scaled by 10**(i-6), both signs, plus 0 and 1."""
    vals = []
    for i in range(7):
        b = np.linspace(0.1, 1, 2 ** i + 1)
        means = (b[:-1] + b[1:]) / 2.0
        vals += list((10.0 ** (i - 6)) * means)
        vals += list(-(10.0 ** (i - 6)) * means)
    vals += [0.0, 1.0]
    assert len(vals) == 256
    return np.sort(np.asarray(vals, dtype=np.float64)).astype(np.float32)


def _nearest(codebook: np.ndarray, x: np.ndarray) -> np.ndarray:
    """Index of the nearest code (codebook sorted ascending)."""
    mid = (codebook[:-1].astype(np.float64) + codebook[1:].astype(np.float64)) / 2
    return np.searchsorted(mid, x.astype(np.float64), side="left").astype(np.uint8)


def quantize(W: np.ndarray, blocksize: int = 64, blocksize2: int = 256):
    """W [N, K] fp32 -> dict(packed uint8 [N*K/2, 1], absmax_q uint8 [nb], absmax2 fp32, code2 fp32 [256],
    offset fp32, shape, blocksize, blocksize2)."""
    W = np.asarray(W, dtype=np.float32)
    flat = W.reshape(-1)
    assert flat.size % blocksize == 0
    blocks = flat.reshape(-1, blocksize)
    absmax = np.abs(blocks).max(axis=1).astype(np.float32)
    safe = np.where(absmax == 0, np.float32(1), absmax)
    idx = _nearest(NF4, blocks / safe[:, None]).reshape(-1)
    packed = ((idx[0::2] << 4) | idx[1::2]).astype(np.uint8).reshape(-1, 1)
    # double quantisation of absmax
    offset = np.float32(absmax.mean())
    a = absmax - offset
    pad = (-a.size) % blocksize2
    ab = np.concatenate([a, np.zeros(pad, np.float32)]).reshape(-1, blocksize2)
    absmax2 = np.abs(ab).max(axis=1).astype(np.float32)
    safe2 = np.where(absmax2 == 0, np.float32(1), absmax2)
    code2 = dynamic_map_8bit()
    absmax_q = _nearest(code2, ab / safe2[:, None]).reshape(-1)[: a.size]
    return {"packed": packed, "absmax_q": absmax_q, "absmax2": absmax2, "code2": code2, "offset": offset,
            "shape": W.shape, "blocksize": blocksize, "blocksize2": blocksize2}


def dequant_absmax(q) -> np.ndarray:
    b = np.arange(q["absmax_q"].size)
    return (q["code2"][q["absmax_q"]] * q["absmax2"][b // q["blocksize2"]]).astype(np.float32) + np.float32(q["offset"])


def dequant(q, out="bf16", code=None):
    """Dense weight [N, K] (row-major, as stored), one RNE rounding of the fp32 product to `out`.  `code`: the 16-entry
    code book the indices refer to (the quant state's `code`; default the NF4 table)."""
    import torch

    NF4 = globals()["NF4"] if code is None else np.asarray(code, dtype=np.float32)  # noqa: N806

    absmax = dequant_absmax(q)
    p = q["packed"].reshape(-1)
    idx = np.empty(p.size * 2, dtype=np.uint8)
    idx[0::2] = p >> 4       # even element: high nibble
    idx[1::2] = p & 0xF
    w = (NF4[idx] * absmax[np.arange(idx.size) // q["blocksize"]]).astype(np.float32).reshape(q["shape"])
    t = torch.from_numpy(w)
    return {"fp32": t, "bf16": t.to(torch.bfloat16), "fp16": t.to(torch.float16)}[out]
