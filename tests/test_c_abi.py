"""The C-ABI library: every symbol declared in include/fmsa.h is exported, and argument validation
returns error codes before any HIP call (so it runs on a machine without a GPU)."""
import ctypes
import os
import re

import pytest

import fmsa_hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "fmsa.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fmsa_[a-z0-9_]+)\s*\(", text)))


def test_header_and_library_agree():
    names = declared_functions()
    assert set(names) == set(fmsa_hip.EXPORTED_SYMBOLS)
    lib = fmsa_hip.lib()
    for n in names:
        assert getattr(lib, n) is not None
    assert lib.fmsa_abi_version() == fmsa_hip.ABI_VERSION  # the binding refuses a library of another version
    assert lib.fmsa_strerror(0) == b"ok" and b"NULL" in lib.fmsa_strerror(-1)


def test_probe_is_a_library_of_its_own():
    """The MFMA-loop probe of `bench.py --yardsticks` is measurement support: the product library does not export it;
    its own library does, and checks its arguments before any HIP call."""
    assert not hasattr(fmsa_hip.lib(), "fmsa_probe_mfma")
    path = os.path.join(ROOT, "fms-acceleration_amd", "lib", "libfmsa_probe.so")
    f = ctypes.CDLL(path).fmsa_probe_mfma
    f.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    assert f(0, 100, 16, None, None, None) == -1
    assert f(2, 100, 16, 0x1000, None, None) == -1      # modes with direct loads need a source
    assert f(4, 100, 16, 0x1000, 0x2000, None) == -2
    assert f(1, 101, 16, 0x1000, None, None) == -2      # two fragment sets used in turn: an even number of iterations
    assert f(1, 100, 0, 0x1000, None, None) == -2


def test_struct_layouts_match_the_header():
    assert ctypes.sizeof(fmsa_hip.GptqWeight) == 72
    assert ctypes.sizeof(fmsa_hip.FwdProj) == 128
    assert ctypes.sizeof(fmsa_hip.BwdProj) == 168
    assert ctypes.sizeof(fmsa_hip.LoraGradJob) == 88
    assert ctypes.sizeof(fmsa_hip.LoraPackJob) == 64


def _w(K=64, N=64, gs=64, q=0x1000, s=0x2000, z=0x3000, g=None, zo=0, order=0):
    return fmsa_hip.GptqWeight(q, s, z, g, K, N, gs, zo, fmsa_hip.WEIGHT_AFFINE, order, None, None)


def _cb(K=64, N=64, gs=64, q=0x1000, code=0x7000, bs=0x8000, g=None, fmt=None):
    """A code-book weight (what fmsa_nf4_prepare produces)."""
    return fmsa_hip.GptqWeight(q, None, None, g, K, N, gs, 0, fmsa_hip.WEIGHT_CODEBOOK if fmt is None else fmt, 0, code, bs)


def test_codebook_weight_validation():
    lib = fmsa_hip.lib()
    f = lib.fmsa_gptq_dequant
    assert f(ctypes.byref(_cb(code=None)), 0, 0x1000, None) == -1
    assert f(ctypes.byref(_cb(bs=None)), 0, 0x1000, None) == -1
    assert f(ctypes.byref(_cb(fmt=2)), 0, 0x1000, None) == -2        # unknown format
    assert f(ctypes.byref(_cb(K=96, gs=64)), 0, 0x1000, None) == -2  # K % group_size
    assert f(ctypes.byref(_cb(g=0x9000)), 0, 0x1000, None) == -5     # no act-order for a code book
    assert f(ctypes.byref(_cb(bs=0x8004)), 0, 0x1000, None) == -3
    assert lib.fmsa_gptq_make_nsz(ctypes.byref(_cb()), 0x1000, None) == -5  # no zero points to tabulate
    # a launch takes projections of one format only
    fw = lambda w: fmsa_hip.FwdProj(w, None, 0, None, None, 0x6000, 64, 0, 0.0)  # noqa: E731
    arr = (fmsa_hip.FwdProj * 2)(fw(_w()), fw(_cb()))
    assert lib.fmsa_gptq_lora_fwd(arr, 2, 0x9000, 64, 8, 0, None, 0, 1, None) == -5
    p = lib.fmsa_nf4_prepare
    nf4 = lambda **kw: fmsa_hip.Nf4Weight(*[kw.get(k, d) for k, d in (  # noqa: E731
        ("packed", 0x1000), ("absmax_q", 0x2000), ("absmax2", 0x3000), ("code2", 0x4000), ("code", None), ("offset", 0.0),
        ("N", 64), ("K", 128), ("blocksize", 64), ("blocksize2", 256))])
    assert p(ctypes.byref(nf4()), None, 0x6000, None) == -1
    assert p(ctypes.byref(nf4(absmax_q=None)), 0x5000, 0x6000, None) == -1
    assert p(ctypes.byref(nf4(K=96)), 0x5000, 0x6000, None) == -2        # K % blocksize
    assert p(ctypes.byref(nf4(blocksize=0)), 0x5000, 0x6000, None) == -2
    assert p(ctypes.byref(nf4()), 0x5004, 0x6000, None) == -3


def test_dequant_validation():
    lib = fmsa_hip.lib()
    f = lib.fmsa_gptq_dequant
    assert f(None, 0, 0x1000, None) == -1
    assert f(ctypes.byref(_w()), 0, None, None) == -1
    assert f(ctypes.byref(_w(q=None)), 0, 0x1000, None) == -1
    assert f(ctypes.byref(_w(K=40)), 0, 0x1000, None) == -2      # K % 32
    assert f(ctypes.byref(_w(N=0)), 0, 0x1000, None) == -2
    assert f(ctypes.byref(_w(zo=2)), 0, 0x1000, None) == -2
    assert f(ctypes.byref(_w(q=0x1004)), 0, 0x1000, None) == -3  # alignment
    assert f(ctypes.byref(_w()), 7, 0x1000, None) == -4          # dtype


def test_fused_forward_validation():
    lib = fmsa_hip.lib()
    f = lib.fmsa_gptq_lora_fwd

    def proj(**kw):
        d = dict(w=_w(), U=0x4000, ldu=16, B=0x5000, bias=None, Y=0x6000, ldy=64, r=16, s=1.0)
        d.update(kw)
        return fmsa_hip.FwdProj(d["w"], d["U"], d["ldu"], d["B"], d["bias"], d["Y"], d["ldy"], d["r"], d["s"])

    def call(p, n=1, X=0x7000, ldx=64, M=8, mode=0, H=None, ldh=0, dt=1):
        arr = (fmsa_hip.FwdProj * 3)(*([p] * 3))
        return f(arr, n, X, ldx, M, mode, H, ldh, dt, None)

    assert call(proj(), X=None) == -1
    assert call(proj(), n=4) == -2
    assert call(proj(), M=0) == -2
    assert call(proj(), dt=2) == -4                       # fp32 is not an activation type
    assert call(proj(), ldx=32) == -2
    assert call(proj(w=_w(g=0x8000))) == -5               # act-order must be repacked first
    assert call(proj(w=_w(gs=24, K=96)), ldx=96) == -5            # group size not a multiple of 16
    assert call(proj(r=12)) == -5
    assert call(proj(U=None)) == -1
    assert call(proj(ldu=8)) == -2                        # U rows shorter than the rank
    assert call(proj(ldu=20)) == -3                       # U rows not 16-byte aligned
    assert call(proj(Y=None)) == -1
    assert call(proj(ldy=32)) == -2
    assert call(proj(), n=1, mode=1) == -2                # SwiGLU needs exactly gate + up
    assert call(proj(), n=2, mode=1, H=None) == -1
    # interleaved words (fmsa_gptq_interleave's output): fp16 activations, whole 64-row stages per group, nothing else
    assert call(proj(w=_w(order=2))) == -2
    assert call(proj(w=_w(order=1)), dt=1) == -5          # bf16 unpacks the checkpoint's order only
    assert call(proj(w=_w(order=1, gs=32)), dt=0) == -5
    assert lib.fmsa_gptq_dequant(ctypes.byref(_w(order=1)), 0, 0x1000, None) == -5   # the forward entry point only
    il = lib.fmsa_gptq_interleave
    assert il(None, 64, 64, 0x2000, None) == -1
    assert il(0x1000, 64, 64, None, None) == -1
    assert il(0x1000, 60, 64, 0x2000, None) == -2
    assert il(0x1000, 64, 66, 0x2000, None) == -2
    assert il(0x1004, 64, 64, 0x2000, None) == -3

    # the flavour that rotates Q / K in its epilogue: the same checks, plus those of the tables and of the head size
    fr = lib.fmsa_gptq_lora_fwd_rope
    assert ctypes.sizeof(fmsa_hip.Rope) == 40

    def rope(**kw):
        d = dict(cos=0xA000, sin=0xB000, ld=64, rows=8, head_dim=64, dtype=1, mask=1)
        d.update(kw)
        return fmsa_hip.Rope(d["cos"], d["sin"], d["ld"], d["rows"], d["head_dim"], d["dtype"], d["mask"])

    def rcall(p, rp, n=1, X=0x7000, ldx=64, M=8, dt=1):
        arr = (fmsa_hip.FwdProj * 3)(*([p] * 3))
        return fr(arr, n, X, ldx, M, ctypes.byref(rp) if rp is not None else None, dt, None)

    assert rcall(proj(), None) == -1
    assert rcall(proj(), rope(cos=None)) == -1
    assert rcall(proj(), rope(), X=None) == -1
    assert rcall(proj(), rope(dtype=0)) == -4              # tables in the other 16-bit type than the activations
    assert rcall(proj(), rope(dtype=7)) == -4
    assert rcall(proj(), rope(head_dim=0)) == -2
    assert rcall(proj(), rope(rows=0)) == -2
    assert rcall(proj(), rope(ld=16)) == -2                # rows shorter than half a head
    assert rcall(proj(), rope(head_dim=96, ld=96)) == -5   # heads would straddle the 256-column tile
    assert rcall(proj(), rope(head_dim=24)) == -5
    assert rcall(proj(), rope(mask=2)) == -2               # names a projection the launch does not have
    assert rcall(proj(), rope(cos=0xA004)) == -3
    assert rcall(proj(), rope(ld=36)) == -3
    assert rcall(proj(), rope(dtype=2, ld=34)) == -3       # fp32 rows must start on 16 bytes too
    assert rcall(proj(), rope(), ldx=32) == -2             # the plain forward's checks still apply
    assert rcall(proj(w=_w(N=96), ldy=96), rope()) == -2   # N is not whole heads
    assert rcall(proj(w=_w(gs=32)), rope()) == -5          # group sizes below the 64-wide K stage
    assert rcall(proj(w=_w(order=1)), rope(dtype=0), dt=0) == -5   # the rotating flavours read the checkpoint's nibble order


def test_bwd_and_skinny_validation():
    lib = fmsa_hip.lib()
    p = fmsa_hip.BwdProj(_w(), 0x9000, 0xA000, 64, 0xB000, 16, 0xC000, None, 0, 16, 1.0)
    arr = (fmsa_hip.BwdProj * 3)(p, p, p)
    f = lib.fmsa_gptq_lora_bwd_dx
    assert f(arr, 1, 8, 0, None, 0, None, None, None, 0, 1, None) == -1       # dX missing
    assert f(arr, 1, 8, 1, None, 0, None, None, None, 0, 1, None) == -1       # e/g/h missing
    assert f(arr, 2, 8, 1, None, 0, 0x1000, 0x2000, 0x3000, 64, 1, None) == -2  # SwiGLU takes one projection
    p2 = fmsa_hip.BwdProj(_w(), None, 0xA000, 64, 0xB000, 16, 0xC000, None, 0, 16, 1.0)
    assert f((fmsa_hip.BwdProj * 1)(p2), 1, 8, 0, 0xD000, 64, None, None, None, 0, 1, None) == -1  # nsz missing
    m1 = fmsa_hip.BwdProj(_w(), 0x9000, 0xA000, 64, 0xB000, 16, 0xC000, 0xE000, 64, 16, 1.0)
    m2 = fmsa_hip.BwdProj(_w(), 0x9000, 0xA000, 64, 0xB000, 16, 0xC000, 0xF000, 64, 16, 1.0)
    assert f((fmsa_hip.BwdProj * 2)(m1, m2), 2, 8, 0, 0xD000, 64, None, None, None, 0, 1, None) == -5  # two masks
    assert lib.fmsa_lora_down(0x1000, 64, 0x2000, 8, 64, 12, 1, 0x3000, 16, None) == -5
    # the flavour with a partial-sum buffer: same argument checks; the size query answers 0 where no buffer is used
    dw, dws = lib.fmsa_lora_down_workspace, lib.fmsa_lora_down_ws
    assert dw(16384, 4096, 16) == 0 and dw(512, 4096, 64) == 0 and dw(4096, 1024, 64) == 0 and dw(0, 4096, 64) == 0
    assert dw(8192, 4096, 16) == 2 * 8192 * 16 * 4
    assert dw(4096, 28672, 64) == 8 * 4096 * 64 * 4 and dw(8192, 4096, 32) == 2 * 8192 * 32 * 4
    assert dw(4096, 8192, 128) == dw(4096, 8192, 64)   # above 64 ranks: 64 at a time through the same buffer
    assert dw(16384, 14336, 32) == 0                   # enough tokens for a workgroup per CU: no column split
    assert dws(None, 64, 0x2000, 8, 64, 16, 1, 0x3000, 16, None, 0, None) == -1
    assert dws(0x1000, 64, 0x2000, 8, 64, 12, 1, 0x3000, 16, None, 0, None) == -5
    assert dws(0x1000, 64, 0x2000, 8, 60, 16, 1, 0x3000, 16, None, 0, None) == -2
    assert dws(0x1000, 64, 0x2000, 8, 64, 16, 1, 0x3000, 8, None, 0, None) == -2
    assert dws(0x1000, 64, 0x2000, 8, 64, 16, 2, 0x3000, 16, None, 0, None) == -4
    assert dws(0x1004, 64, 0x2000, 8, 64, 16, 1, 0x3000, 16, None, 0, None) == -3
    assert dws(0x1000, 64, 0x2000, 8, 64, 16, 1, 0x3000, 16, 0x4004, 1 << 20, None) == -3
    assert lib.fmsa_lora_down(0x1000, 64, 0x2000, 8, 60, 16, 1, 0x3000, 16, None) == -2
    assert lib.fmsa_lora_down(0x1000, 64, 0x2000, 8, 64, 16, 1, 0x3000, 8, None) == -2   # ldout < r
    assert lib.fmsa_lora_grad_workspace(8192, 4096, 16) > 0
    assert lib.fmsa_lora_grad(0x1000, 16, 0x2000, 64, 8, 64, 16, 1.0, 0, 1, 2, 0x3000, None, 0, None) == -6
    # the entry point with the built-in scratch buffer: size and argument errors are reported before any HIP call
    gs = lib.fmsa_lora_grad_static
    assert lib.fmsa_lora_grad_workspace(8192, 14336, 16) <= fmsa_hip.LORA_GRAD_STATIC_BYTES
    assert gs(0x1000, 64, 0x2000, 14336, 8192, 14336, 64, 1.0, 0, 1, 2, 0x3000, None) == -6   # 33 MB of partial sums > 16 MiB
    assert gs(None, 16, 0x2000, 64, 8, 64, 16, 1.0, 0, 1, 2, 0x3000, None) == -1
    assert gs(0x1000, 16, 0x2000, 64, 8, 64, 16, 1.0, 0, 1, 2, None, None) == -1
    assert gs(0x1000, 16, 0x2000, 64, 0, 64, 16, 1.0, 0, 1, 2, 0x3000, None) == -2
    assert gs(0x1000, 16, 0x2000, 32, 8, 64, 16, 1.0, 0, 1, 2, 0x3000, None) == -2             # rows of R shorter than C
    assert gs(0x1000, 16, 0x2000, 64, 8, 64, 12, 1.0, 0, 1, 2, 0x3000, None) == -2
    assert gs(0x1000, 16, 0x2000, 64, 8, 64, 16, 1.0, 0, 2, 2, 0x3000, None) == -4             # fp32 is no activation dtype
    assert gs(0x1000, 16, 0x2000, 64, 8, 64, 16, 1.0, 0, 1, 7, 0x3000, None) == -4
    assert gs(0x1004, 16, 0x2000, 64, 8, 64, 16, 1.0, 0, 1, 2, 0x3000, None) == -3
    J = fmsa_hip.LoraGradJob
    job = lambda **kw: J(**{**dict(L=0x1000, R=0x2000, out=0x3000, ldl=16, ldr=64, C=64, r=16, scale=1.0, transpose_out=0,
                                   out_dtype=2, reserved=0, Wt=None, T=None, ldt=0), **kw})
    gb, gw = lib.fmsa_lora_grad_batch, lib.fmsa_lora_grad_batch_workspace
    two = (J * 2)(job(), job(C=128, ldr=128, r=8))
    assert gw(two, 2, 8) == lib.fmsa_lora_grad_workspace(8, 64, 16) + lib.fmsa_lora_grad_workspace(8, 128, 8)
    assert gw(two, 0, 8) == 0 and gw(two, 9, 8) == 0
    assert gb(None, 1, 8, 1, 0x4000, 1 << 20, None) == -1
    assert gb(two, 0, 8, 1, 0x4000, 1 << 20, None) == -2 and gb(two, 9, 8, 1, 0x4000, 1 << 20, None) == -2
    assert gb(two, 2, 8, 2, 0x4000, 1 << 20, None) == -4                       # fp32 is no activation dtype
    assert gb((J * 2)(job(), job(out=None)), 2, 8, 1, 0x4000, 1 << 20, None) == -1
    assert gb((J * 2)(job(), job(r=12)), 2, 8, 1, 0x4000, 1 << 20, None) == -2
    assert gb((J * 2)(job(), job(ldr=32)), 2, 8, 1, 0x4000, 1 << 20, None) == -2  # rows of R shorter than C
    assert gb((J * 2)(job(), job(out_dtype=7)), 2, 8, 1, 0x4000, 1 << 20, None) == -4
    assert gb((J * 2)(job(), job(L=0x1004)), 2, 8, 1, 0x4000, 1 << 20, None) == -3
    assert gb(two, 2, 8, 1, 0x4000, gw(two, 2, 8) - 1, None) == -6             # workspace one byte short
    with_t = (J * 1)(job(Wt=0x5000, T=0x6000, ldt=16))
    assert gw(with_t, 1, 8) == lib.fmsa_lora_grad_workspace(8, 64, 16) + 1 * 8 * 16 * 4   # + one column block of partial T
    assert gb((J * 1)(job(Wt=0x5000, T=None, ldt=16)), 1, 8, 1, 0x4000, 1 << 20, None) == -1
    assert gb((J * 1)(job(Wt=0x5000, T=0x6000, ldt=8)), 1, 8, 1, 0x4000, 1 << 20, None) == -2
    assert gb((J * 1)(job(Wt=0x5004, T=0x6000, ldt=16)), 1, 8, 1, 0x4000, 1 << 20, None) == -3
    assert gb((J * 2)(job(Wt=0x5000, T=0x6000, ldt=16), job(r=64, ldl=64)), 2, 8, 1, 0x4000, 1 << 20, None) == -5  # T only up to rank 32
    assert gb(two, 2, 8, 1, None, 1 << 20, None) == -6
    assert lib.fmsa_lora_pack(None, 0x1000, 16, 64, 64, 2, 1, None, None, None, None, None) == -1
    assert lib.fmsa_lora_pack(0x1000, 0x2000, 16, 64, 64, 2, 2, None, None, None, None, None) == -4
    P = fmsa_hip.LoraPackJob
    pj = lambda **kw: P(**{**dict(A=0x1000, B=0x2000, A16=0x3000, At16=None, B16=None, Bt16=None, r=16, K=64, N=64, param_dtype=2), **kw})
    pb = lib.fmsa_lora_pack_batch
    assert pb(None, 1, 1, None) == -1 and pb((P * 1)(pj()), 0, 1, None) == -2 and pb((P * 1)(pj()), 5, 1, None) == -2
    assert pb((P * 2)(pj(), pj(B=None)), 2, 1, None) == -1
    assert pb((P * 2)(pj(), pj(N=0)), 2, 1, None) == -2
    assert pb((P * 2)(pj(), pj(param_dtype=5)), 2, 1, None) == -4
    assert pb((P * 2)(pj(), pj()), 2, 2, None) == -4          # fp32 is no activation dtype
    assert lib.fmsa_swiglu_fwd(0x1000, 0x2000, 0x3000, 8, 60, 64, 1, None) == -2
    assert lib.fmsa_gptq_permute_rows(0x1000, 0x2000, 64, 64, 0x1000, None) == -5  # in place


def test_product_path_refuses_cpu_tensors():
    """There is no CPU fallback: the binding raises instead of computing elsewhere."""
    import torch

    with pytest.raises(RuntimeError, match="GPU"):
        fmsa_hip.lora_down(torch.zeros(8, 64, dtype=torch.bfloat16), torch.zeros(8, 64, dtype=torch.bfloat16))
    from fms_acceleration_peft import QuantLinear

    ql = QuantLinear(4, 64, 64, 64, False)
    with pytest.raises(RuntimeError):
        ql(torch.zeros(2, 64, dtype=torch.float16))


def test_norm_rope_validation():
    lib = fmsa_hip.lib()
    f = lib.fmsa_rms_layernorm_fwd
    assert f(None, 64, 0x2000, 8, 64, 1e-5, 0, 1, 1, 0x3000, 64, 0x4000, None) == -1
    assert f(0x1000, 64, 0x2000, 8, 60, 1e-5, 0, 1, 1, 0x3000, 64, 0x4000, None) == -2   # C % 8
    assert f(0x1000, 32, 0x2000, 8, 64, 1e-5, 0, 1, 1, 0x3000, 64, 0x4000, None) == -2   # ldx < C
    assert f(0x1000, 64, 0x2000, 8, 64, 1e-5, 0, 5, 1, 0x3000, 64, 0x4000, None) == -4   # dtype
    assert f(0x1004, 64, 0x2000, 8, 64, 1e-5, 0, 1, 1, 0x3000, 64, 0x4000, None) == -3   # alignment
    b = lib.fmsa_rms_layernorm_bwd
    assert b(0x1000, 64, 0x2000, 64, 0x3000, None, 8, 64, 0, 1, 1, None) == -1           # r missing
    assert b(0x1000, 64, 0x2000, 64, 0x3000, 0x4000, 0, 64, 0, 1, 1, None) == -2
    rp = lib.fmsa_rope_embedding
    assert rp(0x1000, 256, 0x2000, None, 64, 8, 4, 64, 8, 0, 1, 1, None) == -1
    assert rp(0x1000, 256, 0x2000, 0x3000, 64, 8, 4, 24, 8, 0, 1, 1, None) == -2          # head_dim % 16
    assert rp(0x1000, 128, 0x2000, 0x3000, 64, 8, 4, 64, 8, 0, 1, 1, None) == -2          # ldq < heads * head_dim
    assert rp(0x1000, 256, 0x2000, 0x3000, 64, 8, 4, 64, 0, 0, 1, 1, None) == -2          # no cos rows


def test_cross_entropy_validation():
    lib = fmsa_hip.lib()
    f = lib.fmsa_cross_entropy_fwd
    assert f(0x1000, 64, None, 8, 64, 2, 0x2000, 0x3000, None) == -1
    assert f(0x1000, 32, 0x4000, 8, 64, 2, 0x2000, 0x3000, None) == -2   # ld < V
    assert f(0x1000, 64, 0x4000, 8, 64, 9, 0x2000, 0x3000, None) == -4
    b = lib.fmsa_cross_entropy_bwd
    assert b(0x1000, 64, None, 1, 0x2000, 0x4000, 8, 64, 2, None) == -1
    assert b(0x1000, 64, 0x5000, -1, 0x2000, 0x4000, 8, 64, 2, None) == -2
    u = lib.fmsa_cross_entropy_fused
    assert u(0x1000, 64, None, 8, 64, 2, -100, None, 0.0, 0x2000, None) == -1
    assert u(0x1000, 64, 0x4000, 8, 64, 2, -100, None, 0.0, None, None) == -1
    assert u(0x1000, 32, 0x4000, 8, 64, 2, -100, None, 0.0, 0x2000, None) == -2   # ld < V
    assert u(0x1000, 64, 0x4000, 8, 64, 2, -100, None, 1.5, 0x2000, None) == -2   # smoothing outside [0, 1]
    assert u(0x1000, 64, 0x4000, 8, 64, 7, -100, None, 0.0, 0x2000, None) == -4
