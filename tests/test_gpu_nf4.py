"""NF4 path: the dequantisation kernel and the one-time re-layout for the fused kernels bit-exact
against the CPU oracle (whose own parity with bitsandbytes is unpinned: the library is absent and the
reference holds no NF4 vectors), the code-book flavour of the fused GEMM kernels and the
bitsandbytes-flavoured fused operators against the oracle's unfused graph."""
import numpy as np
import pytest
import torch

from oracle import lora as olora
from oracle import nf4 as onf4
from tests.helpers import randn
from tests.model_utils import MaskDropout, make_lora_nf4_linear

pytestmark = pytest.mark.gpu

TOL = 1e-2
_NAME = {torch.float32: "fp32", torch.bfloat16: "bf16", torch.float16: "fp16"}


def _q(t, dtype):
    return t.to(dtype).float()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,K", [(96, 512), (1, 64), (256, 4096), (1000, 192)])
def test_nf4_dequant_bit_exact(N, K, dtype):
    import fmsa_hip

    rng = np.random.default_rng(N * 7 + K)
    W = (rng.standard_normal((N, K)) * rng.uniform(0.005, 0.05, size=(N, 1))).astype(np.float32)
    q = onf4.quantize(W)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    out = fmsa_hip.nf4_dequant(dev(q["packed"]), dev(q["absmax_q"]), dev(q["absmax2"]), dev(q["code2"]),
                               dev(onf4.NF4), float(q["offset"]), (N, K), 64, 256, dtype)
    ref = onf4.dequant(q, _NAME[dtype])
    assert out.shape == (N, K) and out.dtype == dtype
    assert torch.equal(out.cpu(), ref)


def test_nf4_dequant_rejects_bad_shapes():
    import fmsa_hip

    z = torch.zeros(64, dtype=torch.uint8, device="cuda")
    f = torch.zeros(256, device="cuda")
    with pytest.raises(fmsa_hip.FmsaError):
        fmsa_hip.nf4_dequant(z, z, f, f, f[:16], 0.0, (1, 72), 64, 256, torch.bfloat16)  # N*K % blocksize


def test_linear4bit_unfused_forward():
    lin, W, _, _ = make_lora_nf4_linear(256, 128, 8, 16.0, seed=5, device="cuda", bias=True)
    x = randn((4, 10, 256), 1, torch.bfloat16)
    y = lin.base_layer(x.cuda())
    ref = x.float() @ W + lin.base_layer.bias.float().cpu()
    assert olora.max_rel_err(y.cpu(), ref) < TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("B_,S_,K,N,r", [(1, 128, 1024, 2048, 8), (3, 50, 256, 96, 32)])
def test_lora_w(B_, S_, K, N, r, dtype, bias):
    from fms_acceleration_foak.fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_o_v2

    alpha = 2.0 * r
    lin, W, A, B = make_lora_nf4_linear(K, N, r, alpha, seed=3, device="cuda", bias=bias, compute_dtype=dtype)
    x = randn((B_, S_, K), 2, dtype)
    dy = randn((B_, S_, N), 3, dtype)
    xg = x.cuda().requires_grad_(True)
    y = apply_lora_o_v2(lin, xg)
    y.backward(dy.cuda())
    b = lin.base_layer.bias.float().cpu() if bias else None
    y_ref, dx_ref, dA_ref, dB_ref = olora.lora_w_autograd(
        x.float().reshape(-1, K), W, _q(A, dtype), _q(B, dtype), alpha / r, dy.float().reshape(-1, N), b)
    assert y.shape == (B_, S_, N) and y.dtype == dtype
    assert olora.max_rel_err(y.reshape(-1, N), y_ref) < TOL
    assert olora.max_rel_err(xg.grad.reshape(-1, K), dx_ref) < TOL
    gA, gB = lin.lora_A["default"].weight.grad, lin.lora_B["default"].weight.grad
    assert gA.dtype == torch.float32
    assert olora.max_rel_err(gA, dA_ref) < TOL
    assert olora.max_rel_err(gB, dB_ref) < TOL
    assert lin.base_layer.weight.grad is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_lora_qkv(dtype):
    from fms_acceleration_foak.fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_qkv

    Bz, S, K, r, alpha = 2, 96, 1024, 16, 32.0
    Ns = {"q_proj": 1024, "k_proj": 256, "v_proj": 256}
    attn = torch.nn.Module()
    projs = []
    for i, (name, N) in enumerate(Ns.items()):
        lin, W, A, B = make_lora_nf4_linear(K, N, r, alpha, seed=10 + i, device="cuda", compute_dtype=dtype)
        setattr(attn, name, lin)
        projs.append((W, _q(A, dtype), _q(B, dtype), alpha / r))
    x = randn((Bz, S, K), 2, dtype)
    douts = [randn((Bz, S, N), 30 + i, dtype) for i, N in enumerate(Ns.values())]
    xg = x.cuda().requires_grad_(True)
    outs = apply_lora_qkv(attn, xg)
    torch.autograd.backward(outs, [d.cuda() for d in douts])
    outs_ref, dx_ref, grads_ref = olora.lora_qkv_autograd(
        x.float().reshape(-1, K), projs, [d.float().reshape(-1, d.shape[-1]) for d in douts])
    for o, o_ref in zip(outs, outs_ref):
        assert olora.max_rel_err(o.reshape(o_ref.shape), o_ref) < TOL
    assert olora.max_rel_err(xg.grad.reshape(-1, K), dx_ref) < TOL
    for name, (dA_ref, dB_ref) in zip(Ns, grads_ref):
        lin = getattr(attn, name)
        assert olora.max_rel_err(lin.lora_A["default"].weight.grad, dA_ref) < TOL
        assert olora.max_rel_err(lin.lora_B["default"].weight.grad, dB_ref) < TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,H,I,r", [(256, 512, 1024, 16), (100, 256, 704, 8)])
def test_lora_mlp(M, H, I, r, dtype):
    from fms_acceleration_foak.fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_mlp_swiglu

    alpha = 2.0 * r
    mlp = torch.nn.Module()
    ps = []
    for i, (name, K, N) in enumerate((("gate_proj", H, I), ("up_proj", H, I), ("down_proj", I, H))):
        lin, W, A, B = make_lora_nf4_linear(K, N, r, alpha, seed=20 + i, device="cuda", compute_dtype=dtype)
        setattr(mlp, name, lin)
        ps.append((W, _q(A, dtype), _q(B, dtype), alpha / r))
    x = randn((1, M, H), 4, dtype) * 4.0
    dy = randn((1, M, H), 5, dtype)
    xg = x.cuda().requires_grad_(True)
    out = apply_lora_mlp_swiglu(mlp, xg)
    out.backward(dy.cuda())
    out_ref, dx_ref, grads_ref, _ = olora.lora_mlp_autograd(x.float().reshape(-1, H), *ps, dy.float().reshape(-1, H))
    assert olora.max_rel_err(out.reshape(-1, H), out_ref) < TOL
    assert olora.max_rel_err(xg.grad.reshape(-1, H), dx_ref) < TOL
    for name, (dA_ref, dB_ref) in zip(("gate_proj", "up_proj", "down_proj"), grads_ref):
        lin = getattr(mlp, name)
        assert olora.max_rel_err(lin.lora_A["default"].weight.grad, dA_ref) < 2 * TOL, name
        assert olora.max_rel_err(lin.lora_B["default"].weight.grad, dB_ref) < 2 * TOL, name


def test_lora_w_dropout_mask():
    """dX's LoRA term is masked by (dropout(X) != 0) and dA uses the dropped activations
    (fused_ops/unsloth_lora/bnb/fast_lora.py:431-456 of the reference)."""
    from fms_acceleration_foak.fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_o_v2

    dtype, K, N, r, alpha, M = torch.bfloat16, 512, 256, 16, 32.0, 64
    drop = MaskDropout(0.3, (M, K), seed=9)
    lin, W, A, B = make_lora_nf4_linear(K, N, r, alpha, seed=3, device="cuda", dropout=drop.cuda())
    x = randn((M, K), 2, dtype)
    dy = randn((M, N), 3, dtype)
    xg = x.cuda().requires_grad_(True)
    y = apply_lora_o_v2(lin, xg)
    y.backward(dy.cuda())
    xd = x.float() * drop.mask.cpu()
    Aq, Bq, s = _q(A, dtype), _q(B, dtype), alpha / r
    y_ref = x.float() @ W + s * (xd @ Aq.t()) @ Bq.t()
    dx_ref, dA_ref, dB_ref = olora.lora_w_manual(x.float(), W, Aq, Bq, s, dy.float(), xd=xd)
    # lora_w_manual takes W as the matrix of the forward product; its dX uses W^T
    assert olora.max_rel_err(y, y_ref) < TOL
    assert olora.max_rel_err(xg.grad, dx_ref) < TOL
    assert olora.max_rel_err(lin.lora_A["default"].weight.grad, dA_ref) < TOL
    assert olora.max_rel_err(lin.lora_B["default"].weight.grad, dB_ref) < TOL


def _prepared(N, K, seed, blocksize=64):
    """(code-book GptqWeight struct, tensors kept alive, oracle quantisation dict) of a random [N, K] weight."""
    import fmsa_hip

    rng = np.random.default_rng(seed)
    q = onf4.quantize((rng.standard_normal((N, K)) * rng.uniform(0.005, 0.05, size=(N, 1))).astype(np.float32), blocksize)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    qw, bs = fmsa_hip.nf4_prepare(dev(q["packed"]), dev(q["absmax_q"]), dev(q["absmax2"]), dev(q["code2"]), float(q["offset"]),
                                  (N, K), blocksize, 256)
    code = dev(onf4.NF4)
    return fmsa_hip.make_codebook_weight(qw, code, bs, blocksize), (qw, bs, code), q


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,K,blocksize", [(96, 512, 64), (32, 64, 64), (256, 4096, 64), (160, 1024, 128), (64, 256, 32)])
def test_nf4_prepare_bit_exact(N, K, blocksize, dtype):
    """code[q] * block_scale of the re-laid weight == the dequantisation kernel's (and the oracle's) values:
    what the fused kernels feed the MFMA is the library's dense weight, bit for bit."""
    import fmsa_hip

    w, keep, q = _prepared(N, K, N + K, blocksize)
    W = fmsa_hip.weight_dequant(w, torch.device("cuda"), dtype)  # [K, N]
    assert torch.equal(W.cpu(), onf4.dequant(q, _NAME[dtype]).t().contiguous())
    assert keep[0].shape == (K // 8, N) and keep[1].shape == (K // blocksize, N)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("blocksize", [32, 64, 128])
def test_gemm_operands_are_the_dequantised_weight_bit_for_bit(blocksize, dtype):
    """One-hot activations read the MFMA operand straight back: with X = I the forward returns deq(W), with dY = I the
    input gradient returns deq(W)^T, every entry one exact product, so each must equal the oracle's dequantised weight
    rounded once to the activation type, bit for bit: the forward flavour that keeps rounded products as byte planes
    (one block per 64-wide stage, one code book), the one that gathers code values and multiplies (two code-book
    tensors in the launch, or smaller blocks), and the input gradient on both weight layouts."""
    import fmsa_hip

    K, N = 256, 512
    w, keep, q = _prepared(N, K, 11 + blocksize, blocksize)
    want = onf4.dequant(q, _NAME[dtype]).t().contiguous()  # [K, N]
    eye_k, eye_n = torch.eye(K, dtype=dtype, device="cuda"), torch.eye(N, dtype=dtype, device="cuda")
    proj = {"w": w, "U": None, "B": None, "bias": None, "r": 0, "s": 0.0}
    (y,) = fmsa_hip.gptq_lora_fwd(eye_k, [proj])
    assert torch.equal(y.cpu(), want)
    code_twin = keep[2].clone()
    y_a, y_b = fmsa_hip.gptq_lora_fwd(eye_k, [proj, dict(proj, w=fmsa_hip.make_codebook_weight(keep[0], code_twin, keep[1], blocksize))])
    assert torch.equal(y_a.cpu(), want) and torch.equal(y_b.cpu(), want)
    pb = {"w": w, "nsz": None, "dY": eye_n, "T": None, "At": None, "mask_src": None, "r": 0, "s": 0.0}
    layouts = [{}] + ([{"qweight_t": fmsa_hip.gptq_transpose(keep[0])}] if blocksize % 64 == 0 else [])
    for extra in layouts:
        dx = fmsa_hip.gptq_lora_bwd_dx([{**pb, **extra}], N, K)
        assert torch.equal(dx.cpu(), want.t()), sorted(extra)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,N,r,blocksize", [(200, 256, 96, 16, 64), (512, 1024, 512, 8, 64), (64, 1056, 288, 32, 32), (300, 512, 256, 16, 128),
                                               (1, 64, 32, 8, 64), (257, 1344, 608, 24, 64), (31, 96, 1184, 40, 32), (513, 640, 160, 8, 128),
                                               (100, 1152, 896, 16, 64), (7, 2048, 96, 64, 64)])
def test_codebook_kernels(M, K, N, r, blocksize, dtype):
    """Forward (LoRA + bias) and input gradient (LoRA with a mask) of the code-book kernel flavour."""
    import fmsa_hip

    w, keep, q = _prepared(N, K, 3 * N + K, blocksize)
    W = onf4.dequant(q, "fp32").t().contiguous()  # [K, N]
    A, B = olora.make_lora(K, N, r, 5)
    A16, B16 = A.to(dtype), B.to(dtype)
    x = randn((M, K), 6, dtype)
    x[::7, ::5] = 0  # masked entries of the LoRA part of dX
    bias = randn((N,), 7, dtype, scale=0.1)
    s = 2.0
    xd = x.cuda()
    U = fmsa_hip.lora_down(xd, A16.cuda())
    (y,) = fmsa_hip.gptq_lora_fwd(xd, [{"w": w, "U": U, "B": B16.cuda(), "bias": bias.cuda(), "r": r, "s": s}])
    y_ref = olora.lora_linear(x.float(), W, A16.float(), B16.float(), s, bias.float())
    assert olora.max_rel_err(y.cpu(), y_ref) < TOL
    if blocksize % 64 == 0:
        # One block per 64-wide stage and one code book for the launch: the launch above took the flavour that keeps the
        # 16 rounded products of a block and column as byte planes in registers.  A launch over two projections whose code
        # books are different tensors (equal values) stays on the flavour that gathers the code values from the lanes and
        # multiplies: the same products, so the same output bit for bit.
        proj = {"w": w, "U": U, "B": B16.cuda(), "bias": bias.cuda(), "r": r, "s": s}
        code_twin = keep[2].clone()  # (kept alive: the struct holds its address)
        w_twin = fmsa_hip.make_codebook_weight(keep[0], code_twin, keep[1], blocksize)
        y_a, y_b = fmsa_hip.gptq_lora_fwd(xd, [proj, dict(proj, w=w_twin)])
        assert torch.equal(y, y_a) and torch.equal(y, y_b)
    dy = randn((M, N), 8, dtype)
    dyd = dy.cuda()
    T = fmsa_hip.lora_down(dyd, B16.t().contiguous().cuda())
    dx = fmsa_hip.gptq_lora_bwd_dx([{"w": w, "nsz": None, "dY": dyd, "T": T, "At": A16.t().contiguous().cuda(), "mask_src": xd,
                                     "r": r, "s": s}], M, K)
    dx_ref, _, _ = olora.lora_w_manual(x.float(), W, A16.float(), B16.float(), s, dy.float())
    assert olora.max_rel_err(dx.cpu(), dx_ref) < TOL


def test_other_code_book():
    """The kernels take the 16-entry code book from the quant state: with bitsandbytes' FP4 table (not sorted, two
    zeros) in place of NF4 the dense weight, the fused forward (the flavour that keeps rounded products in registers)
    and the input gradient follow the oracle with the same table."""
    import fmsa_hip

    fp4 = (np.array([0, 0.0625, 8, 12, 4, 6, 2, 3, -0.0, -0.0625, -8, -12, -4, -6, -2, -3], dtype=np.float64) / 12).astype(np.float32)
    N, K, M, r, dtype = 256, 512, 200, 16, torch.bfloat16
    w, keep, q = _prepared(N, K, 77)
    code = torch.from_numpy(fp4).cuda()
    w = fmsa_hip.make_codebook_weight(keep[0], code, keep[1], 64)
    Wd = fmsa_hip.weight_dequant(w, torch.device("cuda"), dtype)
    assert torch.equal(Wd.cpu(), onf4.dequant(q, "bf16", code=fp4).t().contiguous())
    W = onf4.dequant(q, "fp32", code=fp4).t().contiguous()
    A, B = olora.make_lora(K, N, r, 5)
    A16, B16 = A.to(dtype), B.to(dtype)
    x = randn((M, K), 6, dtype)
    xd = x.cuda()
    U = fmsa_hip.lora_down(xd, A16.cuda())
    (y,) = fmsa_hip.gptq_lora_fwd(xd, [{"w": w, "U": U, "B": B16.cuda(), "bias": None, "r": r, "s": 2.0}])
    assert olora.max_rel_err(y.cpu(), olora.lora_linear(x.float(), W, A16.float(), B16.float(), 2.0, None)) < TOL
    dy = randn((M, N), 8, dtype)
    T = fmsa_hip.lora_down(dy.cuda(), B16.t().contiguous().cuda())
    dx = fmsa_hip.gptq_lora_bwd_dx([{"w": w, "nsz": None, "dY": dy.cuda(), "T": T, "At": A16.t().contiguous().cuda(), "mask_src": xd,
                                     "r": r, "s": 2.0}], M, K)
    dx_ref, _, _ = olora.lora_w_manual(x.float(), W, A16.float(), B16.float(), 2.0, dy.float())
    assert olora.max_rel_err(dx.cpu(), dx_ref) < TOL


def test_list_style_quant_state_is_accepted():
    """The older bitsandbytes quant state, a list of lists (reference fused_ops/unsloth_lora/utils.py:100-105), gives
    the same dense weight and the same prepared weight as the object form; a list without compressed statistics raises."""
    import fmsa_hip
    from fms_acceleration_foak.fused_ops.unsloth_lora.utils import fast_dequantize
    from fms_acceleration_peft.nf4 import quantize_nf4
    from fmsa_hip.nf4_prepared import PreparedNf4Weight

    W = randn((64, 128), 21, torch.float32).cuda() * 0.02
    packed, qs = quantize_nf4(W, 64, 256, torch.bfloat16)
    as_list = [qs.absmax, qs.shape, qs.dtype, qs.blocksize, [qs.offset, [qs.state2.absmax, qs.state2.code, qs.state2.blocksize, None, None, None, None]],
               "nf4", qs.code]
    assert torch.equal(fast_dequantize(packed, as_list), fast_dequantize(packed, qs))
    a, b = PreparedNf4Weight(packed, as_list), PreparedNf4Weight(packed, qs)
    assert torch.equal(a._keep[0], b._keep[0]) and torch.equal(a._keep[1], b._keep[1])
    with pytest.raises(NotImplementedError, match="compress_statistics"):
        fast_dequantize(packed, [qs.absmax, qs.shape, qs.dtype, qs.blocksize, None, "nf4", qs.code])
