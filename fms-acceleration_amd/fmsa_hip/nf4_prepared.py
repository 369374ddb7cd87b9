"""Per-weight preparation of a bitsandbytes NF4 tensor for the fused kernels, cached on the weight
tensor: the codes re-laid into the word layout the GEMM kernels read and the double-quantised
absmax expanded to one fp32 scale per (block, output column).  The base weight is frozen, so this
happens once; `code[q] * block_scale` reproduces the library's dequantised values bit for bit."""
from __future__ import annotations

import torch

import fmsa_hip


class _State:
    """Attribute view of a quant state."""

    def __init__(self, **kw):
        self.__dict__.update(kw)


def normalize_quant_state(quant_state):
    """bitsandbytes' QuantState object as it is; the older list form
    `[absmax, shape, dtype, blocksize, [offset, [absmax2, code2, blocksize2, ...]], quant_type, code]`
    (what fused_ops/unsloth_lora/utils.py:100-105 of the reference unpacks) as an object with the same
    attribute names."""
    if not isinstance(quant_state, (list, tuple)):
        return quant_state
    if len(quant_state) < 7 or not isinstance(quant_state[4], (list, tuple)) or len(quant_state[4]) != 2:
        raise NotImplementedError("list-style quant state without compressed statistics (compress_statistics=False)")
    absmax, shape, dtype, blocksize, (offset, st2) = quant_state[:5]
    code = quant_state[6]
    if not isinstance(st2, (list, tuple)) or len(st2) < 3:
        raise NotImplementedError("list-style quant state: malformed second-level state")
    state2 = _State(absmax=st2[0], code=st2[1], blocksize=st2[2])
    return _State(absmax=absmax, shape=tuple(shape), dtype=dtype, blocksize=blocksize, offset=offset, state2=state2, code=code)


_code_books = {}


def _shared_code_book(code, device):
    """One device copy per distinct 16-entry code book: weights quantised with the same book (all NF4 weights of a
    model) then hand the kernels the same pointer, which is what lets a launch over several projections keep the
    book in scalar registers.  Read once per prepared weight, on the same path as the re-layout of its codes."""
    host = code.detach().to(device="cpu", dtype=torch.float32).reshape(-1)
    key = (device.type, device.index, tuple(host.tolist()))
    book = _code_books.get(key)
    if book is None:
        book = host.to(device).contiguous()
        _code_books[key] = book
    return book


class PreparedNf4Weight:
    """The C-ABI view (`struct`, code-book format) of one NF4 linear of shape [N, K]."""

    __slots__ = ("struct", "K", "N", "group_size", "perm", "perm_key", "nsz", "_keep", "_twin")

    def __init__(self, W, quant_state):
        quant_state = normalize_quant_state(quant_state)
        state2 = quant_state.state2
        if state2 is None or quant_state.absmax.dtype != torch.uint8:
            raise NotImplementedError("only double-quantised NF4 weights (compress_statistics=True) are supported")
        data = W.data if isinstance(W, torch.nn.Parameter) else W
        if not data.is_cuda:
            raise RuntimeError("fused NF4-LoRA ops need the quantised weight on the GPU")
        N, K = tuple(quant_state.shape)
        bs = int(quant_state.blocksize)
        if K % bs != 0 or bs % 32 != 0 or K % 32 != 0 or N % 32 != 0:
            raise NotImplementedError(
                f"the fused NF4 kernels need in_features % blocksize == 0, blocksize % 32 == 0 and both features "
                f"divisible by 32 (got [{N}, {K}], blocksize {bs})")
        qweight, block_scale = fmsa_hip.nf4_prepare(data.reshape(-1), quant_state.absmax, state2.absmax, state2.code,
                                                    float(quant_state.offset), (N, K), bs, int(state2.blocksize))
        code = _shared_code_book(quant_state.code, data.device)
        self.K, self.N, self.group_size = K, N, bs
        self.perm = self.perm_key = None  # no act-order for NF4
        self.nsz = None   # the input-gradient kernel reads block_scale through the struct
        self._keep = (qweight, block_scale, code)
        self._twin = None
        self.struct = fmsa_hip.make_codebook_weight(qweight, code, block_scale, bs)


def _twin(self):
    """(qweight_t int32 [N/8, K], None, None): the codes packed along N for the input-gradient kernel, built on first use
    (see gptq_prepared.PreparedWeight.twin; the block scales are fp32 already)."""
    if self._twin is None:
        if fmsa_hip.dx_twin_enabled() and self.group_size % 64 == 0:
            self._twin = (fmsa_hip.gptq_transpose(self._keep[0]), None, None)
        else:
            self._twin = (None, None, None)
    return self._twin


PreparedNf4Weight.twin = property(_twin)


def prepare(W, quant_state) -> PreparedNf4Weight:
    data = W.data if isinstance(W, torch.nn.Parameter) else W
    quant_state = normalize_quant_state(quant_state)
    # no float(offset) here: reading a device scalar would synchronise on every call of the hot path
    off = quant_state.offset
    off_key = (off.data_ptr(), off._version) if isinstance(off, torch.Tensor) else float(off)
    key = (data.data_ptr(), data._version, quant_state.absmax.data_ptr(), quant_state.absmax._version,
           off_key, tuple(quant_state.shape), int(quant_state.blocksize))
    cached = getattr(W, "_fmsa_prepared", None)
    if cached is None or cached[0] != key:
        cached = (key, PreparedNf4Weight(W, quant_state))
        W._fmsa_prepared = cached
    return cached[1]
