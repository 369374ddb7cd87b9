"""ctypes binding of libfmsa_hip.so (C ABI declared in include/fmsa.h).

The library is built in-tree by ``build_hip.py`` and loaded from ``../lib``.  Nothing here falls
back to another implementation: if the library is missing, or a call returns an error code, a
RuntimeError is raised.  torch is used only for device memory (tensors) and the current stream.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p
from typing import Optional, Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libfmsa_hip.so")

F16, BF16, F32 = 0, 1, 2
FWD_LINEAR, FWD_SWIGLU = 0, 1
BWD_LINEAR, BWD_SWIGLU = 0, 1

_DTYPE_ENUM = {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32}

EXPORTED_SYMBOLS = (
    "fmsa_strerror",
    "fmsa_abi_version",
    "fmsa_gptq_dequant",
    "fmsa_gptq_permute_rows",
    "fmsa_permute_cols",
    "fmsa_lora_down",
    "fmsa_lora_down_workspace",
    "fmsa_lora_down_ws",
    "fmsa_lora_grad_workspace",
    "fmsa_lora_grad",
    "fmsa_lora_grad_batch_workspace",
    "fmsa_lora_grad_batch",
    "fmsa_lora_grad_static",
    "fmsa_gptq_lora_fwd",
    "fmsa_gptq_lora_fwd_rope",
    "fmsa_gptq_lora_bwd_dx",
    "fmsa_swiglu_fwd",
    "fmsa_swiglu_bwd",
    "fmsa_gptq_make_nsz",
    "fmsa_gptq_transpose",
    "fmsa_gptq_interleave",
    "fmsa_nf4_dequant",
    "fmsa_nf4_prepare",
    "fmsa_lora_pack",
    "fmsa_lora_pack_batch",
    "fmsa_rms_layernorm_fwd",
    "fmsa_rms_layernorm_bwd",
    "fmsa_rope_embedding",
    "fmsa_cross_entropy_fwd",
    "fmsa_cross_entropy_bwd",
    "fmsa_cross_entropy_fused",
)


class GptqWeight(Structure):
    _fields_ = [
        ("qweight", c_void_p),
        ("scales", c_void_p),
        ("qzeros", c_void_p),
        ("g_idx", c_void_p),
        ("K", c_int32),
        ("N", c_int32),
        ("group_size", c_int32),
        ("zero_offset", c_int32),
        ("format", c_int32),
        ("nibble_order", c_int32),
        ("code", c_void_p),
        ("block_scale", c_void_p),
    ]


WEIGHT_AFFINE, WEIGHT_CODEBOOK = 0, 1


class Rope(Structure):
    _fields_ = [
        ("cos", c_void_p),
        ("sin", c_void_p),
        ("ld", c_int64),
        ("rows", c_int32),
        ("head_dim", c_int32),
        ("dtype", c_int32),
        ("proj_mask", c_int32),
    ]


class Nf4Weight(Structure):
    _fields_ = [
        ("packed", c_void_p),
        ("absmax_q", c_void_p),
        ("absmax2", c_void_p),
        ("code2", c_void_p),
        ("code", c_void_p),
        ("offset", c_float),
        ("N", c_int32),
        ("K", c_int32),
        ("blocksize", c_int32),
        ("blocksize2", c_int32),
    ]


class LoraGradJob(Structure):
    """fmsa_lora_grad_job: one scale * L[M, r]^T @ R[M, C] of a batch."""

    _fields_ = [
        ("L", c_void_p),
        ("R", c_void_p),
        ("out", c_void_p),
        ("ldl", c_int64),
        ("ldr", c_int64),
        ("C", c_int32),
        ("r", c_int32),
        ("scale", c_float),
        ("transpose_out", c_int32),
        ("out_dtype", c_int32),
        ("reserved", c_int32),
        ("Wt", c_void_p),
        ("T", c_void_p),
        ("ldt", c_int64),
    ]


class LoraPackJob(Structure):
    """fmsa_lora_pack_job: one adapter of a batched pack."""

    _fields_ = [
        ("A", c_void_p),
        ("B", c_void_p),
        ("A16", c_void_p),
        ("At16", c_void_p),
        ("B16", c_void_p),
        ("Bt16", c_void_p),
        ("r", c_int32),
        ("K", c_int32),
        ("N", c_int32),
        ("param_dtype", c_int32),
    ]


class FwdProj(Structure):
    _fields_ = [
        ("w", GptqWeight),
        ("U", c_void_p),
        ("ldu", c_int64),
        ("B", c_void_p),
        ("bias", c_void_p),
        ("Y", c_void_p),
        ("ldy", c_int64),
        ("r", c_int32),
        ("s", c_float),
    ]


class BwdProj(Structure):
    _fields_ = [
        ("w", GptqWeight),
        ("nsz", c_void_p),
        ("dY", c_void_p),
        ("lddy", c_int64),
        ("T", c_void_p),
        ("ldt", c_int64),
        ("At", c_void_p),
        ("mask_src", c_void_p),
        ("ldmask", c_int64),
        ("r", c_int32),
        ("s", c_float),
        ("qweight_t", c_void_p),
        ("scale_f32", c_void_p),
        ("negzp_f16", c_void_p),
    ]


_lib = None


ABI_VERSION = 9  # include/fmsa.h as this binding mirrors it (fmsa_abi_version of the library must agree)


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python fms-acceleration_amd/build_hip.py` "
            "(there is no fallback path for the fused quantised-LoRA kernels)"
        )
    L = ctypes.CDLL(LIB_PATH)
    L.fmsa_strerror.restype = ctypes.c_char_p
    L.fmsa_strerror.argtypes = [c_int]
    L.fmsa_abi_version.restype = c_int
    if L.fmsa_abi_version() != ABI_VERSION:
        # struct layouts and signatures below are those of ABI_VERSION: a library of another version would read them wrong
        raise RuntimeError(f"{LIB_PATH} has ABI version {L.fmsa_abi_version()}, this binding is written for {ABI_VERSION}: "
                           "rebuild it with `python fms-acceleration_amd/build_hip.py`")
    L.fmsa_gptq_dequant.argtypes = [POINTER(GptqWeight), c_int, c_void_p, c_void_p]
    L.fmsa_gptq_permute_rows.argtypes = [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p]
    L.fmsa_permute_cols.argtypes = [c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int64, c_void_p]
    L.fmsa_lora_down.argtypes = [c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int64, c_void_p]
    L.fmsa_lora_down_workspace.restype = c_size_t
    L.fmsa_lora_down_workspace.argtypes = [c_int, c_int, c_int]
    L.fmsa_lora_down_ws.argtypes = [c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int64, c_void_p, c_size_t,
                                    c_void_p]
    L.fmsa_lora_grad_workspace.restype = c_size_t
    L.fmsa_lora_grad_workspace.argtypes = [c_int, c_int, c_int]
    L.fmsa_lora_grad.argtypes = [c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_int, c_float, c_int, c_int, c_int,
                                 c_void_p, c_void_p, c_size_t, c_void_p]
    L.fmsa_lora_grad_batch_workspace.restype = c_size_t
    L.fmsa_lora_grad_batch_workspace.argtypes = [POINTER(LoraGradJob), c_int, c_int]
    L.fmsa_lora_grad_batch.argtypes = [POINTER(LoraGradJob), c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]
    L.fmsa_lora_grad_static.argtypes = [c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_int, c_float, c_int, c_int, c_int,
                                        c_void_p, c_void_p]
    L.fmsa_gptq_lora_fwd.argtypes = [POINTER(FwdProj), c_int, c_void_p, c_int64, c_int, c_int, c_void_p, c_int64,
                                     c_int, c_void_p]
    L.fmsa_gptq_lora_fwd_rope.argtypes = [POINTER(FwdProj), c_int, c_void_p, c_int64, c_int, POINTER(Rope), c_int, c_void_p]
    L.fmsa_gptq_lora_bwd_dx.argtypes = [POINTER(BwdProj), c_int, c_int, c_int, c_void_p, c_int64, c_void_p, c_void_p,
                                        c_void_p, c_int64, c_int, c_void_p]
    L.fmsa_swiglu_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int, c_void_p]
    L.fmsa_swiglu_bwd.argtypes = [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int, c_void_p]
    L.fmsa_gptq_make_nsz.argtypes = [POINTER(GptqWeight), c_void_p, c_void_p]
    L.fmsa_gptq_transpose.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p]
    L.fmsa_gptq_interleave.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p]
    L.fmsa_nf4_dequant.argtypes = [POINTER(Nf4Weight), c_int, c_void_p, c_void_p]
    L.fmsa_nf4_prepare.argtypes = [POINTER(Nf4Weight), c_void_p, c_void_p, c_void_p]
    L.fmsa_lora_pack.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_void_p]
    L.fmsa_lora_pack_batch.argtypes = [POINTER(LoraPackJob), c_int, c_int, c_void_p]
    L.fmsa_rms_layernorm_fwd.argtypes = [c_void_p, c_int64, c_void_p, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p,
                                         c_int64, c_void_p, c_void_p]
    L.fmsa_rms_layernorm_bwd.argtypes = [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                         c_int, c_void_p]
    L.fmsa_rope_embedding.argtypes = [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int, c_int,
                                      c_int, c_void_p]
    L.fmsa_cross_entropy_fwd.argtypes = [c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
    L.fmsa_cross_entropy_bwd.argtypes = [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]
    L.fmsa_cross_entropy_fused.argtypes = [c_void_p, c_int64, c_void_p, c_int, c_int, c_int, c_int64, c_void_p, c_float, c_void_p, c_void_p]
    for name in EXPORTED_SYMBOLS:
        getattr(L, name)  # AttributeError here means the library is stale: rebuild it
    _lib = L
    return L


class FmsaError(RuntimeError):
    def __init__(self, fn: str, code: int):
        msg = lib().fmsa_strerror(code).decode()
        super().__init__(f"{fn} failed with code {code}: {msg}")
        self.code = code


def _check(fn: str, code: int):
    if code != 0:
        raise FmsaError(fn, code)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else c_void_p(t.data_ptr())


def _stream(t: torch.Tensor):
    if not t.is_cuda:
        raise RuntimeError("libfmsa_hip kernels need tensors on the GPU (there is no CPU implementation)")
    return c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def act_enum(dtype: torch.dtype) -> int:
    if dtype not in (torch.float16, torch.bfloat16):
        raise TypeError(f"activations must be float16 or bfloat16, got {dtype}")
    return _DTYPE_ENUM[dtype]


def make_weight(qweight, scales, qzeros, g_idx, group_size: int, zero_offset: int = 0, nibble_order: int = 0) -> GptqWeight:
    """GptqWeight from QuantLinear buffers.  g_idx=None declares the identity assignment.  nibble_order=1 declares
    that qweight is gptq_interleave's output (forward entry point, fp16 activations, group_size % 64 == 0 only)."""
    K = qweight.shape[0] * 8
    N = qweight.shape[1]
    assert qweight.dtype == torch.int32 and qzeros.dtype == torch.int32 and scales.dtype == torch.float16
    assert qweight.is_contiguous() and qzeros.is_contiguous() and scales.is_contiguous()
    return GptqWeight(
        qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(),
        None if g_idx is None else g_idx.data_ptr(), K, N, int(group_size), int(zero_offset), WEIGHT_AFFINE, int(nibble_order), None, None,
    )


def make_codebook_weight(qweight, code, block_scale, group_size: int) -> GptqWeight:
    """GptqWeight of a 4-bit code-book weight in the word layout (what nf4_prepare returns):
    W[k, n] = code[q[k, n]] * block_scale[k // group_size, n]."""
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    assert qweight.dtype == torch.int32 and code.dtype == torch.float32 and block_scale.dtype == torch.float32
    assert qweight.is_contiguous() and code.is_contiguous() and block_scale.is_contiguous()
    assert code.numel() == 16 and block_scale.shape == (K // group_size, N)
    return GptqWeight(qweight.data_ptr(), None, None, None, K, N, int(group_size), 0, WEIGHT_CODEBOOK, 0,
                      code.data_ptr(), block_scale.data_ptr())


def weight_dequant(w: GptqWeight, device, out_dtype=torch.float16):
    """Dense [K, N] of any GptqWeight (affine or code-book), one rounding to out_dtype."""
    out = torch.empty((w.K, w.N), dtype=out_dtype, device=device)
    _check("fmsa_gptq_dequant", lib().fmsa_gptq_dequant(ctypes.byref(w), _DTYPE_ENUM[out_dtype], _ptr(out), _stream(out)))
    return out


# ---- thin tensor-level wrappers ------------------------------------------------------------------
def gptq_dequant(qweight, scales, qzeros, g_idx, group_size, zero_offset=0, out_dtype=torch.float16):
    """W [K, N] = scales[g] * (q - z - zero_offset), one RNE rounding to out_dtype."""
    w = make_weight(qweight, scales, qzeros, g_idx, group_size, zero_offset)
    out = torch.empty((w.K, w.N), dtype=out_dtype, device=qweight.device)
    _check("fmsa_gptq_dequant", lib().fmsa_gptq_dequant(ctypes.byref(w), _DTYPE_ENUM[out_dtype], _ptr(out), _stream(out)))
    return out


def gptq_make_nsz(w: GptqWeight, device) -> torch.Tensor:
    """fp32 [G, N] table -scale * (zero + zero_offset) read by the input-gradient kernel."""
    G = (w.K + w.group_size - 1) // w.group_size
    out = torch.empty((G, w.N), dtype=torch.float32, device=device)
    _check("fmsa_gptq_make_nsz", lib().fmsa_gptq_make_nsz(ctypes.byref(w), _ptr(out), _stream(out)))
    return out


def gptq_permute_rows(qweight, perm):
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    out = torch.empty_like(qweight)
    _check("fmsa_gptq_permute_rows",
           lib().fmsa_gptq_permute_rows(_ptr(qweight), _ptr(perm), K, N, _ptr(out), _stream(out)))
    return out


def permute_cols(x2d, perm, gather: bool):
    M, C = x2d.shape
    out = torch.empty((M, C), dtype=x2d.dtype, device=x2d.device)
    _check("fmsa_permute_cols",
           lib().fmsa_permute_cols(_ptr(x2d), x2d.stride(0), _ptr(perm), M, C, int(gather), act_enum(x2d.dtype),
                                   _ptr(out), out.stride(0), _stream(out)))
    return out


def lora_down(x2d, wd, out=None):
    """out [M, r] = x2d [M, C] @ wd [r, C]^T.  `out` may be a column slice of a wider buffer."""
    M, C = x2d.shape
    r = wd.shape[0]
    assert wd.shape[1] == C and wd.is_contiguous() and wd.dtype == x2d.dtype and x2d.stride(1) == 1
    if out is None:
        out = torch.empty((M, r), dtype=x2d.dtype, device=x2d.device)
    assert out.shape == (M, r) and out.stride(1) == 1 and out.dtype == x2d.dtype
    nbytes = lib().fmsa_lora_down_workspace(M, C, r)
    ws = _workspace(nbytes, x2d.device) if nbytes else None
    _check("fmsa_lora_down_ws", lib().fmsa_lora_down_ws(_ptr(x2d), x2d.stride(0), _ptr(wd), M, C, r, act_enum(x2d.dtype), _ptr(out),
                                                        out.stride(0), _ptr(ws), 0 if ws is None else ws.numel(), _stream(out)))
    return out


_ws_cache = {}


def _workspace(nbytes: int, device) -> torch.Tensor:
    """Partial-sum buffer of the adapter-gradient launches, one per (device, stream): launches on one stream
    are ordered and may share it, launches on two streams of one device must not."""
    key = (device.type, device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _ws_cache.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _ws_cache[key] = ws
    return ws


def lora_grad(L, R, scale: float, transpose_out: bool, out_dtype=torch.float32):
    """scale * L[M, r]^T @ R[M, C] -> [r, C] (or [C, r] when transpose_out)."""
    M, r = L.shape
    C = R.shape[1]
    assert R.shape[0] == M and L.stride(1) == 1 and R.stride(1) == 1 and L.dtype == R.dtype
    out = torch.empty((C, r) if transpose_out else (r, C), dtype=out_dtype, device=R.device)
    nbytes = lib().fmsa_lora_grad_workspace(M, C, r)
    ws = _workspace(nbytes, R.device)
    _check("fmsa_lora_grad",
           lib().fmsa_lora_grad(_ptr(L), L.stride(0), _ptr(R), R.stride(0), M, C, r, float(scale), int(transpose_out),
                                act_enum(R.dtype), _DTYPE_ENUM[out_dtype], _ptr(out), _ptr(ws), ws.numel(), _stream(out)))
    return out


LORA_GRAD_STATIC_BYTES = 16 << 20


def lora_grad_static(L, R, scale: float, transpose_out: bool, out):
    """lora_grad through the entry point that allocates nothing: the partial sums go to a buffer inside the
    library's device image (LORA_GRAD_STATIC_BYTES; larger requests raise), `out` is the caller's.  Calls that
    overlap on one GPU share that buffer and race."""
    M, r = L.shape
    C = R.shape[1]
    assert R.shape[0] == M and L.stride(1) == 1 and R.stride(1) == 1 and L.dtype == R.dtype
    assert out.is_contiguous() and tuple(out.shape) == ((C, r) if transpose_out else (r, C))
    assert L.device == R.device == out.device
    with torch.cuda.device(out.device):  # the library uses the buffer of the thread's current device
        _check("fmsa_lora_grad_static",
               lib().fmsa_lora_grad_static(_ptr(L), L.stride(0), _ptr(R), R.stride(0), M, C, r, float(scale), int(transpose_out),
                                           act_enum(R.dtype), _DTYPE_ENUM[out.dtype], _ptr(out), _stream(out)))
    return out


LORA_GRAD_MAX_JOBS = 8


LORA_GRAD_T_MAX_RANK = 32  # fmsa_lora_grad_batch computes T next to the gradient only up to this rank


def lora_grad_batch(jobs):
    """jobs: (L, R, scale, transpose_out, out_dtype[, Wt, T_out]) tuples over the same M tokens; returns
    the list of scale * L^T @ R, each as lora_grad would give it, from one launch of each pass per
    LORA_GRAD_MAX_JOBS jobs.  A job with Wt [r, C] and T_out [M, r] (may be a column slice) also gets
    T_out = R @ Wt^T from the same pass over R (all ranks of such a call <= LORA_GRAD_T_MAX_RANK)."""
    outs = []
    for i in range(0, len(jobs), LORA_GRAD_MAX_JOBS):
        chunk = jobs[i : i + LORA_GRAD_MAX_JOBS]
        M = chunk[0][0].shape[0]
        arr = (LoraGradJob * len(chunk))()
        for q, job in enumerate(chunk):
            L, R, scale, tr, out_dtype = job[:5]
            Wt, T_out = job[5:7] if len(job) > 5 else (None, None)
            r, C = L.shape[1], R.shape[1]
            assert L.shape[0] == M and R.shape[0] == M and L.stride(1) == 1 and R.stride(1) == 1
            assert L.dtype == R.dtype == chunk[0][1].dtype
            if Wt is not None:
                assert Wt.shape == (r, C) and Wt.is_contiguous() and Wt.dtype == R.dtype
                assert T_out.shape == (M, r) and T_out.stride(1) == 1 and T_out.dtype == R.dtype
            out = torch.empty((C, r) if tr else (r, C), dtype=out_dtype, device=R.device)
            outs.append(out)
            arr[q] = LoraGradJob(_ptr(L), _ptr(R), _ptr(out), L.stride(0), R.stride(0), C, r, float(scale), int(tr),
                                 _DTYPE_ENUM[out_dtype], 0, _ptr(Wt), _ptr(T_out), 0 if T_out is None else T_out.stride(0))
        R0 = chunk[0][1]
        ws = _workspace(lib().fmsa_lora_grad_batch_workspace(arr, len(chunk), M), R0.device)
        _check("fmsa_lora_grad_batch",
               lib().fmsa_lora_grad_batch(arr, len(chunk), M, act_enum(R0.dtype), _ptr(ws), ws.numel(), _stream(R0)))
    return outs


def gptq_lora_fwd(x2d, projs: Sequence[dict], mode: int = FWD_LINEAR, rope=None):
    """projs: dicts with keys w (GptqWeight), U, B, bias (tensors or None), r, s.
    Returns the list of outputs Y_p [M, N_p]; in SWIGLU mode returns (e, g, h).
    rope = (cos2d, sin2d, head_dim, proj_mask): LINEAR mode only; the projections whose bit is set in proj_mask
    leave with the rotary embedding applied (token row m takes row m % cos2d.shape[0] of the tables)."""
    M = x2d.shape[0]
    arr = (FwdProj * len(projs))()
    outs = []
    for i, p in enumerate(projs):
        w = p["w"]
        y = torch.empty((M, w.N), dtype=x2d.dtype, device=x2d.device)
        outs.append(y)
        U = p.get("U") if p["r"] else None
        assert U is None or U.stride(1) == 1
        arr[i] = FwdProj(w, _ptr(U), 0 if U is None else U.stride(0), _ptr(p.get("B")) if p["r"] else None,
                         _ptr(p.get("bias")), _ptr(y), y.stride(0), int(p["r"]), float(p["s"] or 0.0))
    h = None
    if mode == FWD_SWIGLU:
        h = torch.empty_like(outs[0])
    if rope is not None:
        cos2d, sin2d, head_dim, proj_mask = rope
        assert mode == FWD_LINEAR and cos2d.shape == sin2d.shape and cos2d.dtype == sin2d.dtype
        assert cos2d.stride(1) == 1 and sin2d.stride(1) == 1 and cos2d.stride(0) == sin2d.stride(0) and cos2d.is_cuda
        if cos2d.dim() != 2 or cos2d.shape[1] < int(head_dim) // 2:
            raise ValueError("cos / sin must be [positions, >= head_dim / 2]")
        desc = Rope(_ptr(cos2d), _ptr(sin2d), cos2d.stride(0), cos2d.shape[0], int(head_dim), _DTYPE_ENUM[cos2d.dtype], int(proj_mask))
        _check("fmsa_gptq_lora_fwd_rope",
               lib().fmsa_gptq_lora_fwd_rope(arr, len(projs), _ptr(x2d), x2d.stride(0), M, ctypes.byref(desc),
                                             act_enum(x2d.dtype), _stream(x2d)))
        return outs
    _check("fmsa_gptq_lora_fwd",
           lib().fmsa_gptq_lora_fwd(arr, len(projs), _ptr(x2d), x2d.stride(0), M, mode, _ptr(h),
                                    0 if h is None else h.stride(0), act_enum(x2d.dtype), _stream(x2d)))
    if mode == FWD_SWIGLU:
        return outs[0], outs[1], h
    return outs


def gptq_lora_bwd_dx(projs: Sequence[dict], M: int, K: int, mode: int = BWD_LINEAR, e=None, g=None):
    """projs: dicts with keys w, nsz, dY, T, At, mask_src, r, s and optionally qweight_t, scale_f32, negzp_f16 (the
    weight's transposed twin and its tables, see gptq_transpose and gptq_negzp_f16).  LINEAR mode returns dX [M, K]; SWIGLU mode overwrites e <- d_g,
    g <- d_e and returns h."""
    arr = (BwdProj * len(projs))()
    ref = projs[0]["dY"]
    for i, p in enumerate(projs):
        dy = p["dY"]
        assert dy.stride(1) == 1
        ms = p.get("mask_src")
        T = p.get("T") if p["r"] else None
        assert T is None or T.stride(1) == 1
        arr[i] = BwdProj(p["w"], _ptr(p["nsz"]), _ptr(dy), dy.stride(0), _ptr(T), 0 if T is None else T.stride(0),
                         _ptr(p.get("At")) if p["r"] else None, _ptr(ms), 0 if ms is None else ms.stride(0),
                         int(p["r"]), float(p["s"] or 0.0), _ptr(p.get("qweight_t")), _ptr(p.get("scale_f32")),
                         _ptr(p.get("negzp_f16")))
    if mode == BWD_SWIGLU:
        h = torch.empty_like(e)
        _check("fmsa_gptq_lora_bwd_dx",
               lib().fmsa_gptq_lora_bwd_dx(arr, len(projs), M, mode, None, 0, _ptr(e), _ptr(g), _ptr(h), e.stride(0),
                                           act_enum(ref.dtype), _stream(ref)))
        return h
    dx = torch.empty((M, K), dtype=ref.dtype, device=ref.device)
    _check("fmsa_gptq_lora_bwd_dx",
           lib().fmsa_gptq_lora_bwd_dx(arr, len(projs), M, mode, _ptr(dx), dx.stride(0), None, None, None, 0,
                                       act_enum(ref.dtype), _stream(ref)))
    return dx


def dx_twin_enabled() -> bool:
    """Whether prepared weights build the transposed twin the input-gradient kernel prefers (one more packed copy
    of every frozen weight, 4 bits per weight, plus fp32 scales).  FMSA_DX_TWIN=0 keeps the checkpoint layout only."""
    return os.environ.get("FMSA_DX_TWIN", "1") != "0"


def fwd_interleaved_enabled() -> bool:
    """Whether prepared weights build the interleaved copy the forward kernel's packed-half unpack reads for fp16
    activations (one more packed copy of every frozen weight, 4 bits per weight).  FMSA_FWD_INTERLEAVED=0 keeps the
    checkpoint layout only."""
    return os.environ.get("FMSA_FWD_INTERLEAVED", "1") != "0"


def gptq_negzp_f16(qzeros, N: int, zero_offset: int = 0):
    """fp16 [G, N] = -(1024 + zero point + zero_offset), exact in fp16: the offset table of the packed-half unpack
    (fmsa_bwd_proj.negzp_f16)."""
    shifts = torch.arange(0, 32, 4, device=qzeros.device, dtype=torch.int64)
    z = ((qzeros.to(torch.int64).unsqueeze(-1) >> shifts) & 0xF).reshape(qzeros.shape[0], -1)[:, :N]
    return (-(1024 + z + int(zero_offset))).to(torch.float16).contiguous()


def gptq_interleave(qweight):
    """The packed weight [K/8, N] with the nibbles of every word interleaved (element 2p at position p, element 2p + 1 at
    position 4 + p): what the forward kernel's packed-half unpack reads (GptqWeight.nibble_order = 1, fp16 activations)."""
    K8, N = qweight.shape
    assert qweight.dtype == torch.int32 and qweight.is_contiguous() and N % 4 == 0
    out = torch.empty_like(qweight)
    _check("fmsa_gptq_interleave", lib().fmsa_gptq_interleave(_ptr(qweight), K8 * 8, N, _ptr(out), _stream(qweight)))
    return out


def gptq_transpose(qweight):
    """The transposed twin [N/8, K] of a packed weight [K/8, N]: word [n8, k] holds q[k, 8 n8 + e], element 2p at nibble
    position p, element 2p + 1 at position 4 + p."""
    K8, N = qweight.shape
    assert qweight.dtype == torch.int32 and qweight.is_contiguous() and N % 8 == 0
    out = torch.empty((N // 8, K8 * 8), dtype=torch.int32, device=qweight.device)
    _check("fmsa_gptq_transpose", lib().fmsa_gptq_transpose(_ptr(qweight), K8 * 8, N, _ptr(out), _stream(qweight)))
    return out


def swiglu_fwd(e, g):
    """h = silu(e) * g with the reference's rounding points (standalone kernel)."""
    M, I = e.shape
    assert e.stride() == g.stride() and e.stride(1) == 1
    h = torch.empty_like(e)
    _check("fmsa_swiglu_fwd", lib().fmsa_swiglu_fwd(_ptr(e), _ptr(g), _ptr(h), M, I, e.stride(0), act_enum(e.dtype), _stream(e)))
    return h


def swiglu_bwd(dh, e, g):
    """In place: e <- d_g, g <- d_e; returns h."""
    M, I = e.shape
    assert e.stride() == g.stride() and e.stride(1) == 1 and dh.stride(1) == 1
    h = torch.empty_like(e)
    _check("fmsa_swiglu_bwd", lib().fmsa_swiglu_bwd(_ptr(dh), dh.stride(0), _ptr(e), _ptr(g), _ptr(h), M, I, e.stride(0),
                                                    act_enum(e.dtype), _stream(e)))
    return h


def nf4_dequant(packed, absmax_q, absmax2, code2, code, offset: float, shape, blocksize: int, blocksize2: int,
                out_dtype=torch.bfloat16):
    """Dense [N, K] weight of a bitsandbytes NF4 tensor with double-quantised absmax."""
    N, K = shape
    w = Nf4Weight(packed.data_ptr(), absmax_q.data_ptr(), absmax2.data_ptr(), code2.data_ptr(), code.data_ptr(),
                  float(offset), N, K, blocksize, blocksize2)
    out = torch.empty((N, K), dtype=out_dtype, device=packed.device)
    _check("fmsa_nf4_dequant", lib().fmsa_nf4_dequant(ctypes.byref(w), _DTYPE_ENUM[out_dtype], _ptr(out), _stream(out)))
    return out


def nf4_prepare(packed, absmax_q, absmax2, code2, offset: float, shape, blocksize: int, blocksize2: int):
    """(qweight int32 [K/8, N], block_scale fp32 [K / blocksize, N]) of an NF4 tensor [N, K]: the
    one-time re-layout the fused kernels read (see make_codebook_weight)."""
    N, K = shape
    w = Nf4Weight(packed.data_ptr(), absmax_q.data_ptr(), absmax2.data_ptr(), code2.data_ptr(), None, float(offset), N, K,
                  blocksize, blocksize2)
    qweight = torch.empty((K // 8, N), dtype=torch.int32, device=packed.device)
    block_scale = torch.empty((K // blocksize, N), dtype=torch.float32, device=packed.device)
    _check("fmsa_nf4_prepare", lib().fmsa_nf4_prepare(ctypes.byref(w), _ptr(qweight), _ptr(block_scale), _stream(qweight)))
    return qweight, block_scale


LORA_PACK_MAX_JOBS = 4


def lora_pack_batch(adapters, act_dtype):
    """adapters: (lora_A.weight [r, K], lora_B.weight [N, r], A16_out or None) triples (fp32 / bf16 / fp16
    parameters).  Returns one (A16 [r, K], At16 [K, r], B16 [N, r], Bt16 [r, N]) per adapter in `act_dtype`,
    from one launch per LORA_PACK_MAX_JOBS adapters.  `A16_out` (contiguous [r, K]) lets the caller place A16
    inside a larger stacked matrix."""
    outs, jobs = [], []
    for A, B, A16_out in adapters:
        if not (A.is_cuda and B.is_cuda):
            raise RuntimeError("fmsa_hip needs GPU tensors")
        A, B = A.detach(), B.detach()
        if A.dtype != B.dtype:
            B = B.to(A.dtype)
        A = A if A.is_contiguous() else A.contiguous()
        B = B if B.is_contiguous() else B.contiguous()
        r, K = A.shape
        N = B.shape[0]
        own_a = A16_out is None
        buf = torch.empty(r * K * (2 if own_a else 1) + 2 * r * N, dtype=act_dtype, device=A.device)
        o = 0
        if own_a:
            A16_out, o = buf[: r * K].view(r, K), r * K
        assert A16_out.shape == (r, K) and A16_out.is_contiguous() and A16_out.dtype == act_dtype
        At16 = buf[o : o + r * K].view(K, r)
        B16 = buf[o + r * K : o + r * K + N * r].view(N, r)
        Bt16 = buf[o + r * K + N * r :].view(r, N)
        outs.append((A16_out, At16, B16, Bt16))
        jobs.append((A, B, LoraPackJob(_ptr(A), _ptr(B), _ptr(A16_out), _ptr(At16), _ptr(B16), _ptr(Bt16), r, K, N,
                                       _DTYPE_ENUM[A.dtype])))
    for i in range(0, len(jobs), LORA_PACK_MAX_JOBS):
        chunk = jobs[i : i + LORA_PACK_MAX_JOBS]
        arr = (LoraPackJob * len(chunk))(*[j for _, _, j in chunk])
        _check("fmsa_lora_pack_batch", lib().fmsa_lora_pack_batch(arr, len(chunk), act_enum(act_dtype), _stream(chunk[0][0])))
    return outs


def lora_pack(A, B, act_dtype, A16_out=None):
    """lora_pack_batch for one adapter."""
    return lora_pack_batch([(A, B, A16_out)], act_dtype)[0]


def rms_layernorm_fwd(x2d, weight, eps: float, gemma: bool = False):
    """(Y [M, C] in x2d's dtype, r [M] fp32 = 1 / rms) of an RMS layer norm over the rows of x2d."""
    if not (x2d.is_cuda and weight.is_cuda):
        raise RuntimeError("fmsa_hip needs GPU tensors")
    M, C = x2d.shape
    assert x2d.stride(1) == 1 and weight.is_contiguous() and weight.numel() == C
    y = torch.empty((M, C), dtype=x2d.dtype, device=x2d.device)
    r = torch.empty(M, dtype=torch.float32, device=x2d.device)
    _check("fmsa_rms_layernorm_fwd",
           lib().fmsa_rms_layernorm_fwd(_ptr(x2d), x2d.stride(0), _ptr(weight), M, C, float(eps), int(gemma), _DTYPE_ENUM[x2d.dtype],
                                        _DTYPE_ENUM[weight.dtype], _ptr(y), y.stride(0), _ptr(r), _stream(x2d)))
    return y, r


def rms_layernorm_bwd(dy2d, x2d, weight, r, gemma: bool = False):
    """Overwrites dy2d with dX and returns it."""
    M, C = x2d.shape
    assert dy2d.shape == (M, C) and dy2d.stride(1) == 1 and x2d.stride(1) == 1 and dy2d.dtype == x2d.dtype
    _check("fmsa_rms_layernorm_bwd",
           lib().fmsa_rms_layernorm_bwd(_ptr(dy2d), dy2d.stride(0), _ptr(x2d), x2d.stride(0), _ptr(weight), _ptr(r), M, C, int(gemma),
                                        _DTYPE_ENUM[x2d.dtype], _DTYPE_ENUM[weight.dtype], _stream(x2d)))
    return dy2d


def rope_embedding_(q2d, cos2d, sin2d, n_heads: int, head_dim: int, backward: bool = False):
    """In place on q2d [M, n_heads * head_dim]; row m uses row m % cos2d.shape[0] of cos / sin."""
    if not (q2d.is_cuda and cos2d.is_cuda and sin2d.is_cuda):
        raise RuntimeError("fmsa_hip needs GPU tensors")
    assert q2d.stride(1) == 1 and cos2d.stride(1) == 1 and cos2d.stride() == sin2d.stride() and cos2d.dtype == sin2d.dtype
    _check("fmsa_rope_embedding",
           lib().fmsa_rope_embedding(_ptr(q2d), q2d.stride(0), _ptr(cos2d), _ptr(sin2d), cos2d.stride(0), q2d.shape[0], n_heads,
                                     head_dim, cos2d.shape[0], int(backward), _DTYPE_ENUM[q2d.dtype], _DTYPE_ENUM[cos2d.dtype],
                                     _stream(q2d)))
    return q2d


def cross_entropy_fwd(logits2d, labels):
    """(losses [M] fp32, logsumexp [M] fp32); labels int64 [M], -100 ignored."""
    if not (logits2d.is_cuda and labels.is_cuda):
        raise RuntimeError("fmsa_hip needs GPU tensors")
    M, V = logits2d.shape
    assert logits2d.stride(1) == 1 and labels.dtype == torch.int64 and labels.is_contiguous() and labels.numel() == M
    losses = torch.empty(M, dtype=torch.float32, device=logits2d.device)
    lse = torch.empty(M, dtype=torch.float32, device=logits2d.device)
    _check("fmsa_cross_entropy_fwd", lib().fmsa_cross_entropy_fwd(_ptr(logits2d), logits2d.stride(0), _ptr(labels), M, V,
                                                                  _DTYPE_ENUM[logits2d.dtype], _ptr(losses), _ptr(lse), _stream(logits2d)))
    return losses, lse


def cross_entropy_bwd_(logits2d, dlosses, lse, labels):
    """Overwrites logits2d with the gradient and returns it; dlosses [M] fp32 (any stride, 0 included)."""
    M, V = logits2d.shape
    assert dlosses.dtype == torch.float32 and dlosses.numel() == M and dlosses.dim() == 1
    _check("fmsa_cross_entropy_bwd", lib().fmsa_cross_entropy_bwd(_ptr(logits2d), logits2d.stride(0), _ptr(dlosses), dlosses.stride(0),
                                                                  _ptr(lse), _ptr(labels), M, V, _DTYPE_ENUM[logits2d.dtype],
                                                                  _stream(logits2d)))
    return logits2d


def cross_entropy_fused_(logits2d, labels, scale=None, label_smoothing=0.0, ignore_index=-100, losses_out=None):
    """Overwrites logits2d with scale * d(loss)/d(logits) and returns (losses [M] fp32, already scaled;
    logits2d).  `scale` is a 1-element fp32 GPU tensor (None = 1)."""
    if not (logits2d.is_cuda and labels.is_cuda):
        raise RuntimeError("fmsa_hip needs GPU tensors")
    M, V = logits2d.shape
    assert logits2d.stride(1) == 1 and labels.dtype == torch.int64 and labels.is_contiguous() and labels.numel() == M
    assert scale is None or (scale.is_cuda and scale.dtype == torch.float32 and scale.numel() == 1)
    losses = losses_out if losses_out is not None else torch.empty(M, dtype=torch.float32, device=logits2d.device)
    assert losses.dtype == torch.float32 and losses.is_contiguous() and losses.numel() == M
    _check("fmsa_cross_entropy_fused",
           lib().fmsa_cross_entropy_fused(_ptr(logits2d), logits2d.stride(0), _ptr(labels), M, V, _DTYPE_ENUM[logits2d.dtype],
                                          int(ignore_index), _ptr(scale) if scale is not None else None, float(label_smoothing),
                                          _ptr(losses), _stream(logits2d)))
    return losses, logits2d
