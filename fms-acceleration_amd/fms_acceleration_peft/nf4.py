"""bitsandbytes-style NF4 base layer: the data layout the `bitsandbytes` fused operators read.

Stand-ins for `bitsandbytes.nn.Linear4bit`, `Params4bit` and `functional.QuantState` with the
attribute names the reference's operators use (fused-ops-and-kernels/.../unsloth_lora/utils.py:53-141):
`layer.weight` (packed uint8 [N*K/2, 1]) carrying `.quant_state` with `absmax` (uint8 when double
quantised), `shape`, `dtype`, `blocksize`, `code`, `offset` and `state2` (`absmax` fp32, `code`,
`blocksize`).  bitsandbytes is not installed where this is built; a real Linear4bit exposes the same
attributes and is accepted by the fused operators as is.

`quantize_4bit` builds such a weight from a dense matrix (blockwise absmax, nearest of the 16 codes
of the NF4 or FP4 book, even element in the high nibble; absmax minus its mean re-quantised to 8
bits in blocks of 256) -- how synthetic 4-bit checkpoints are made for tests and benchmarks, and how
the plugin's loader quantises a dense checkpoint.
"""
from __future__ import annotations

import torch
from torch import nn

NF4_CODE = [-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
            -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
            0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
            0.7229568362236023, 1.0]


# bitsandbytes' FP4 book (functional.get_4bit_type("fp4")): sign bit, then E2M1-like magnitudes in the library's own
# code order, divided by the largest (12).  Not sorted: index i is what the packed nibble holds.
FP4_CODE = [v / 12.0 for v in (0.0, 0.0625, 8.0, 12.0, 4.0, 6.0, 2.0, 3.0, -0.0, -0.0625, -8.0, -12.0, -4.0, -6.0, -2.0, -3.0)]

CODE_BOOKS = {"nf4": NF4_CODE, "fp4": FP4_CODE}


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
    """Index of the nearest entry; the book need not be sorted (ties go to the smaller value)."""
    order = torch.argsort(codebook, stable=True)
    srt = codebook[order]
    mid = (srt[:-1].double() + srt[1:].double()) / 2
    return order[torch.bucketize(x.double(), mid, right=False)]


@torch.no_grad()
def quantize_4bit(W: torch.Tensor, blocksize: int = 64, blocksize2: int = 256, dtype=torch.bfloat16, quant_type: str = "nf4"):
    """W [N, K] -> (packed uint8 [N*K/2, 1], QuantState)."""
    W = W.float()
    dev = W.device
    code = torch.tensor(CODE_BOOKS[quant_type], dtype=torch.float32, device=dev)
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
    state = QuantState(absmax_q, W.shape, dtype, blocksize, code, offset.reshape(()), QuantState2(absmax2, code2, blocksize2),
                       quant_type=quant_type)
    return packed, state


def quantize_nf4(W, blocksize=64, blocksize2=256, dtype=torch.bfloat16):
    return quantize_4bit(W, blocksize, blocksize2, dtype, "nf4")


class Params4bit(nn.Parameter):
    """Packed 4-bit weight; `quant_state` travels on the parameter object."""

    def __new__(cls, data, quant_state=None):
        self = torch.Tensor._make_subclass(cls, data, False)
        self.quant_state = quant_state
        return self

    def __deepcopy__(self, memo):
        import copy  # pylint: disable=import-outside-toplevel

        # nn.Parameter's own __deepcopy__ would call the constructor with (data, requires_grad)
        twin = type(self)(self.data.clone(memory_format=torch.preserve_format), copy.deepcopy(self.quant_state, memo))
        memo[id(self)] = twin
        return twin


class Linear4bitFunction(torch.autograd.Function):
    """y = x @ deq(W)^T, dx = dy @ deq(W) for a frozen 4-bit weight (what bitsandbytes' MatMul4Bit computes:
    dequantise, then a dense matmul; no gradient for the weight).  16-bit activations go through the fused
    dequant-GEMM kernels with the adapter switched off (r = 0): the codes are looked up on their way into the MFMA
    and no dense matrix is written."""

    @staticmethod
    def forward(ctx, x, weight, quant_state):
        import fmsa_hip
        from fmsa_hip.nf4_prepared import prepare

        w = prepare(weight, quant_state)
        ctx.w = w
        x2 = x if x.is_contiguous() else x.contiguous()
        (y,) = fmsa_hip.gptq_lora_fwd(x2, [{"w": w.struct, "U": None, "B": None, "bias": None, "r": 0, "s": 0.0}])
        return y

    @staticmethod
    def backward(ctx, dy):
        import fmsa_hip

        w = ctx.w
        dy2 = dy if dy.is_contiguous() else dy.contiguous()
        dx = fmsa_hip.gptq_lora_bwd_dx(
            [{"w": w.struct, "nsz": w.nsz, "dY": dy2, "T": None, "At": None, "mask_src": None, "r": 0, "s": 0.0,
              "qweight_t": w.twin[0], "scale_f32": w.twin[1], "negzp_f16": w.twin[2]}], dy2.shape[0], w.K)
        return dx, None, None


class Linear4bit(nn.Module):
    """4-bit (NF4 / FP4 code book) linear.  `forward` is the module-level path without LoRA fusion: the fused
    dequant-GEMM kernels with r = 0 for 16-bit activations, dequantise (HIP kernel) + matmul otherwise."""

    def __init__(self, in_features, out_features, bias=False, compute_dtype=torch.bfloat16):
        super().__init__()
        self.in_features, self.out_features, self.compute_dtype = in_features, out_features, compute_dtype
        self.weight = Params4bit(torch.zeros((in_features * out_features // 2, 1), dtype=torch.uint8))
        self.bias = nn.Parameter(torch.zeros(out_features, dtype=compute_dtype), requires_grad=False) if bias else None

    @classmethod
    def from_dense(cls, weight: torch.Tensor, bias=None, compute_dtype=torch.bfloat16, blocksize=64, blocksize2=256,
                   quant_type="nf4"):
        N, K = weight.shape
        self = cls(K, N, bias is not None, compute_dtype)
        packed, state = quantize_4bit(weight, blocksize, blocksize2, compute_dtype, quant_type)
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
        qs = self.weight.quant_state
        fused = (x.is_cuda and x.dtype in (torch.float16, torch.bfloat16) and qs is not None and qs.state2 is not None
                 and self.in_features % qs.blocksize == 0 and qs.blocksize % 32 == 0
                 and self.in_features % 32 == 0 and self.out_features % 32 == 0)
        if fused:
            out = Linear4bitFunction.apply(x.reshape(-1, x.shape[-1]), self.weight, qs)
            out = out.reshape(x.shape[:-1] + (self.out_features,))
        else:
            out = x @ self.dequantize(x.dtype).t()
        return out + self.bias.to(out.dtype) if self.bias is not None else out
