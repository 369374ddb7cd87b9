"""bitsandbytes-style NF4 base layer: the data layout the `bitsandbytes` fused operators read.

Stand-ins for `bitsandbytes.nn.Linear4bit`, `Params4bit` and `functional.QuantState` with the
attribute names the reference's operators use (fused-ops-and-kernels/.../unsloth_lora/utils.py:53-141):
`layer.weight` (packed uint8 [N*K/2, 1]) carrying `.quant_state` with `absmax` (uint8 when double
quantised), `shape`, `dtype`, `blocksize`, `code`, `offset` and `state2` (`absmax` fp32, `code`,
`blocksize`).  bitsandbytes is not installed where this is built; a real Linear4bit exposes the same
attributes and is accepted by the fused operators as is.

`quantize_nf4` builds such a weight from a dense matrix (blockwise absmax, nearest of the 16 NF4
codes, even element in the high nibble; absmax minus its mean re-quantised to 8 bits in blocks of
256) -- how synthetic NF4 checkpoints are made for tests and benchmarks.
"""
from __future__ import annotations

import torch
from torch import nn

NF4_CODE = [-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
            -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
            0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
            0.7229568362236023, 1.0]


def dynamic_map_8bit() -> torch.Tensor:
    """Signed dynamic 8-bit code book for the absmax statistics (256 sorted values in [-1, 1])."""
    vals = []
    for i in range(7):
        b = torch.linspace(0.1, 1, 2 ** i + 1, dtype=torch.float64)
        means = (b[:-1] + b[1:]) / 2
        vals += [means * 10.0 ** (i - 6), -means * 10.0 ** (i - 6)]
    vals.append(torch.tensor([0.0, 1.0], dtype=torch.float64))
    return torch.sort(torch.cat(vals)).values.to(torch.float32)


class QuantState2:
    def __init__(self, absmax, code, blocksize):
        self.absmax, self.code, self.blocksize = absmax, code, blocksize

    def to(self, device):
        self.absmax, self.code = self.absmax.to(device), self.code.to(device)
        return self


class QuantState:
    def __init__(self, absmax, shape, dtype, blocksize, code, offset, state2, quant_type="nf4"):
        self.absmax, self.shape, self.dtype, self.blocksize = absmax, torch.Size(shape), dtype, blocksize
        self.code, self.offset, self.state2, self.quant_type = code, offset, state2, quant_type
        self.nested = state2 is not None

    def to(self, device):
        self.absmax, self.code, self.offset = self.absmax.to(device), self.code.to(device), self.offset.to(device)
        if self.state2 is not None:
            self.state2.to(device)
        return self


def _nearest(codebook: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    mid = (codebook[:-1].double() + codebook[1:].double()) / 2
    return torch.bucketize(x.double(), mid, right=False)


@torch.no_grad()
def quantize_nf4(W: torch.Tensor, blocksize: int = 64, blocksize2: int = 256, dtype=torch.bfloat16):
    """W [N, K] -> (packed uint8 [N*K/2, 1], QuantState)."""
    W = W.float()
    dev = W.device
    code = torch.tensor(NF4_CODE, dtype=torch.float32, device=dev)
    blocks = W.reshape(-1, blocksize)
    absmax = blocks.abs().amax(dim=1)
    safe = torch.where(absmax == 0, torch.ones_like(absmax), absmax)
    idx = _nearest(code, blocks / safe[:, None]).reshape(-1).to(torch.uint8)
    packed = ((idx[0::2] << 4) | idx[1::2]).reshape(-1, 1)
    offset = absmax.mean()
    a = absmax - offset
    pad = (-a.numel()) % blocksize2
    ab = torch.cat([a, a.new_zeros(pad)]).reshape(-1, blocksize2)
    absmax2 = ab.abs().amax(dim=1)
    safe2 = torch.where(absmax2 == 0, torch.ones_like(absmax2), absmax2)
    code2 = dynamic_map_8bit().to(dev)
    absmax_q = _nearest(code2, ab / safe2[:, None]).reshape(-1)[: a.numel()].to(torch.uint8)
    state = QuantState(absmax_q, W.shape, dtype, blocksize, code, offset.reshape(()), QuantState2(absmax2, code2, blocksize2))
    return packed, state


class Params4bit(nn.Parameter):
    """Packed 4-bit weight; `quant_state` travels on the parameter object."""

    def __new__(cls, data, quant_state=None):
        self = torch.Tensor._make_subclass(cls, data, False)
        self.quant_state = quant_state
        return self


class Linear4bit(nn.Module):
    """NF4 linear.  `forward` is the unfused path: dequantise (HIP kernel) then matmul."""

    def __init__(self, in_features, out_features, bias=False, compute_dtype=torch.bfloat16):
        super().__init__()
        self.in_features, self.out_features, self.compute_dtype = in_features, out_features, compute_dtype
        self.weight = Params4bit(torch.zeros((in_features * out_features // 2, 1), dtype=torch.uint8))
        self.bias = nn.Parameter(torch.zeros(out_features, dtype=compute_dtype), requires_grad=False) if bias else None

    @classmethod
    def from_dense(cls, weight: torch.Tensor, bias=None, compute_dtype=torch.bfloat16, blocksize=64, blocksize2=256):
        N, K = weight.shape
        self = cls(K, N, bias is not None, compute_dtype)
        packed, state = quantize_nf4(weight, blocksize, blocksize2, compute_dtype)
        self.weight = Params4bit(packed, state)
        if bias is not None:
            self.bias.data.copy_(bias)
        return self

    def _apply(self, fn, recurse=True):
        state = self.weight.quant_state
        super()._apply(fn, recurse)
        if not isinstance(self.weight, Params4bit):
            self.weight = Params4bit(self.weight.data, state)
        self.weight.quant_state = state
        if state is not None:
            state.to(self.weight.device)
        return self

    def dequantize(self, dtype=None):
        """Dense [N, K] weight in `dtype` (default: the quant state's dtype)."""
        import fmsa_hip

        qs = self.weight.quant_state
        return fmsa_hip.nf4_dequant(self.weight.data, qs.absmax, qs.state2.absmax, qs.state2.code, qs.code,
                                    float(qs.offset), tuple(qs.shape), qs.blocksize, qs.state2.blocksize,
                                    dtype or qs.dtype)

    def forward(self, x):
        out = x @ self.dequantize(x.dtype).t()
        return out + self.bias.to(out.dtype) if self.bias is not None else out
