"""Per-weight preparation for the fused GPTQ kernels, cached on the qweight tensor: the C-ABI view
of one QuantLinear, the one-time row repack of act-order weights, and the fp32 offset table the
input-gradient kernel reads.  Shared by the fused LoRA operators and by QuantLinear's own forward."""
from __future__ import annotations

import torch

import fmsa_hip


class PreparedWeight:
    """The C-ABI view of one QuantLinear.  For an act-order g_idx the packed rows are re-ordered
    once (fmsa_gptq_permute_rows) so that the group of row k' is k' // group_size; `perm` then
    maps the kernels' row order back to the model's: row k' of the repacked weight is row
    perm[k'] of the original.  Projections quantised on the same input (q, k, v; gate, up) get the
    same order from act-order GPTQ (it sorts by the diagonal of the input's Hessian): `perm_key`
    lets their callers see that and keep them in one launch."""

    __slots__ = ("struct", "K", "N", "group_size", "perm", "perm_key", "nsz", "_keep", "_zero_offset", "_columns", "col_inv", "_row_inv",
                 "_twin", "_interleaved")

    def __init__(self, qweight, scales, qzeros, g_idx, bits):
        if bits != 4:
            raise NotImplementedError(f"the gfx950 fused kernels cover 4-bit GPTQ only (got bits={bits})")
        if not qweight.is_cuda:
            raise RuntimeError("fused GPTQ-LoRA ops need the quantised weight on the GPU")
        K, N, G = qweight.shape[0] * 8, qweight.shape[1], scales.shape[0]
        if K % G != 0:
            raise NotImplementedError(f"in_features {K} is not a multiple of the number of groups {G}")
        gs = K // G
        zero_offset = int(getattr(qzeros, "offset", 0) or 0)
        qweight, scales, qzeros = qweight.contiguous(), scales.contiguous(), qzeros.contiguous()
        ident = torch.arange(K, device=g_idx.device, dtype=torch.int64) // gs
        g64 = g_idx.to(torch.int64)
        g64 = torch.where(g64 < 0, g64 + G, g64)
        perm = None
        self.perm_key = None  # hashable identity of the row order: weights with equal keys can share one launch
        if not torch.equal(g64, ident):
            perm64 = torch.argsort(g64, stable=True)
            if not torch.equal(g64[perm64], ident):
                raise NotImplementedError("act-order g_idx with groups of unequal size is not supported")
            perm = perm64.to(torch.int32).contiguous()
            self.perm_key = hash(perm.cpu().numpy().tobytes())
            qweight = fmsa_hip.gptq_permute_rows(qweight, perm)
        self.K, self.N, self.group_size, self.perm = K, N, gs, perm
        self._zero_offset = zero_offset
        self._row_inv = None
        self._columns = {}    # column-permuted twins, by the key of the permutation
        self.col_inv = None   # set on such a twin: natural column n is column col_inv[n] of the twin
        self._finish(qweight, scales, qzeros)

    def _finish(self, qweight, scales, qzeros):
        self._keep = (qweight, scales, qzeros)
        self._twin = None
        self._interleaved = None
        self.struct = fmsa_hip.make_weight(qweight, scales, qzeros, None, self.group_size, self._zero_offset)
        # -scale * zero per (group, column), fp32: read by the input-gradient kernel (frozen weight,
        # so it is built once)
        self.nsz = fmsa_hip.gptq_make_nsz(self.struct, qweight.device)

    @property
    def twin(self):
        """(qweight_t int32 [N/8, K], scale_f32 [G, N], negzp_f16 [G, N]) for the input-gradient kernel, built on first
        use (the weight is frozen): the nibbles packed along N, so that a lane's word is its MFMA fragment as in the
        forward kernel, the scales widened once, and the fp16 offsets of the packed-half unpack (fp16 activations).
        (None, None, None) when switched off or when a group does not hold whole 64-column wave tiles (the kernel then
        reads the checkpoint layout)."""
        if self._twin is None:
            if fmsa_hip.dx_twin_enabled() and self.group_size % 64 == 0:
                qweight, scales, qzeros = self._keep
                self._twin = (fmsa_hip.gptq_transpose(qweight), scales.to(torch.float32).contiguous(),
                              fmsa_hip.gptq_negzp_f16(qzeros, self.N, self._zero_offset))
            else:
                self._twin = (None, None, None)
        return self._twin

    def interleaved_ok(self, dtype) -> bool:
        """Whether the forward kernel's packed-half unpack applies: fp16 activations, groups in whole 64-row stages."""
        return dtype == torch.float16 and self.group_size % 64 == 0 and fmsa_hip.fwd_interleaved_enabled()

    @property
    def struct_interleaved(self):
        """The C-ABI view of a copy of the packed weight whose words hold their nibbles interleaved (nibble_order 1),
        built on first use: the forward kernel unpacks it with packed-half arithmetic (fp16 activations only)."""
        if self._interleaved is None:
            qweight, scales, qzeros = self._keep
            q_il = fmsa_hip.gptq_interleave(qweight)
            struct = fmsa_hip.make_weight(q_il, scales, qzeros, None, self.group_size, self._zero_offset, nibble_order=1)
            self._interleaved = (struct, q_il)
        return self._interleaved[0]

    @property
    def row_inv(self):
        """Inverse of `perm` (int64): the model's row k is row row_inv[k] of the repacked weight."""
        if self._row_inv is None:
            self._row_inv = torch.argsort(self.perm.long())
        return self._row_inv

    def with_columns(self, col_perm, key):
        """The same weight with its output columns re-ordered: column n' of the twin is column col_perm[n'] of
        this one (built once per permutation).  An MLP whose down projection is act-order lets gate and up
        produce e, g and h directly in the row order the down projection's repacked weight wants."""
        twin = self._columns.get(key)
        if twin is None:
            qweight, scales, qzeros = self._keep
            idx = col_perm.long()
            shifts = torch.arange(0, 32, 4, device=qzeros.device, dtype=torch.int64)
            z = ((qzeros.to(torch.int64).unsqueeze(-1) >> shifts) & 0xF).reshape(qzeros.shape[0], -1)[:, idx]
            zw = (z.reshape(qzeros.shape[0], -1, 8) << shifts).sum(-1)
            zw = torch.where(zw >= 2**31, zw - 2**32, zw).to(torch.int32)
            twin = object.__new__(PreparedWeight)
            twin.K, twin.N, twin.group_size, twin.perm, twin.perm_key = self.K, self.N, self.group_size, self.perm, self.perm_key
            twin._zero_offset, twin._columns, twin._row_inv = self._zero_offset, {}, None
            twin.col_inv = torch.argsort(idx)
            twin._finish(qweight[:, idx].contiguous(), scales[:, idx].contiguous(), zw.contiguous())
            self._columns[key] = twin
        return twin


def prepare(qweight, scales, qzeros, g_idx, bits) -> PreparedWeight:
    key = (qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(), g_idx.data_ptr(), g_idx._version,
           qweight._version, scales._version, qzeros._version, int(getattr(qzeros, "offset", 0) or 0))
    cached = getattr(qweight, "_fmsa_prepared", None)
    if cached is None or cached[0] != key:
        cached = (key, PreparedWeight(qweight, scales, qzeros, g_idx, bits))
        qweight._fmsa_prepared = cached
    return cached[1]


