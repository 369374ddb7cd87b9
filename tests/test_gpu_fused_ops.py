"""The fused autograd functions (through the C ABI) against the CPU oracle's unfused graph."""
import pytest
import torch

from oracle import lora as olora
from tests.helpers import randn
from tests.model_utils import MaskDropout, make_lora_gptq_linear

pytestmark = pytest.mark.gpu

TOL = 1e-2  # max |out - ref| / max |ref| against the fp32 oracle, per tensor


def _q(t, dtype):
    """fp32 value of a tensor after rounding to the activation dtype (what the kernels see)."""
    return t.to(dtype).float()


@pytest.fixture(params=["own_pass", "with_dB"], autouse=True)
def t_product_route(request, monkeypatch):
    """The backward forms T = dY B either in its own pass over dY or inside the dB launch (the route large
    shapes take): every test of this file runs both ways."""
    from fms_acceleration_foak.fused_ops.unsloth_lora import fused_core

    if request.param == "with_dB":
        monkeypatch.setattr(fused_core, "FUSE_T_MIN_BYTES", 0)
    return request.param


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("B_,S_,K,N,r", [(1, 128, 2048, 2048, 8), (2, 256, 512, 1024, 16), (3, 50, 256, 96, 32)])
def test_lora_w(B_, S_, K, N, r, dtype, act_order):
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_o_v2

    alpha = 2.0 * r
    lin, W, A, B = make_lora_gptq_linear(K, N, r, alpha, seed=3, act_order=act_order, device="cuda",
                                         group_size=128 if K % 128 == 0 else 64)
    x = randn((B_, S_, K), 2, dtype)
    dy = randn((B_, S_, N), 3, dtype)
    xg = x.cuda().requires_grad_(True)
    y = apply_lora_o_v2(lin, xg)
    y.backward(dy.cuda())
    y_ref, dx_ref, dA_ref, dB_ref = olora.lora_w_autograd(
        x.float().reshape(-1, K), W, _q(A, dtype), _q(B, dtype), alpha / r, dy.float().reshape(-1, N))
    assert y.shape == (B_, S_, N) and y.dtype == dtype
    assert olora.max_rel_err(y.reshape(-1, N), y_ref) < TOL
    assert olora.max_rel_err(xg.grad.reshape(-1, K), dx_ref) < TOL
    gA, gB = lin.lora_A["default"].weight.grad, lin.lora_B["default"].weight.grad
    assert gA.shape == A.shape and gB.shape == B.shape and gA.dtype == torch.float32
    assert olora.max_rel_err(gA, dA_ref) < TOL
    assert olora.max_rel_err(gB, dB_ref) < TOL
    # the frozen base gets no gradient
    assert all(not b.requires_grad for b in lin.base_layer.buffers())


# act_order "shared": one permutation for the projections that read the same input (what act-order GPTQ produces,
# since it sorts by the input's Hessian diagonal): they stay in one launch; True: one permutation per projection
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act_order", [False, True, "shared"])
def test_lora_qkv(dtype, act_order):
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_qkv

    Bz, S, K, r, alpha = 2, 96, 1024, 16, 32.0
    Ns = {"q_proj": 1024, "k_proj": 256, "v_proj": 256}
    attn = torch.nn.Module()
    refs = {}
    for i, (name, N) in enumerate(Ns.items()):
        lin, W, A, B = make_lora_gptq_linear(K, N, r, alpha, seed=10 + i, act_order=act_order, device="cuda",
                                             order_seed=99 if act_order == "shared" else None)
        setattr(attn, name, lin)
        refs[name] = (W, _q(A, dtype), _q(B, dtype), alpha / r)
    x = randn((Bz, S, K), 2, dtype)
    douts = [randn((Bz, S, N), 30 + i, dtype) for i, N in enumerate(Ns.values())]
    xg = x.cuda().requires_grad_(True)
    Q, Kt, V = apply_lora_qkv(attn, xg)
    # dK reaches the function non-contiguous in the reference's attention (a transposed view)
    torch.autograd.backward([Q, Kt, V], [d.cuda() for d in douts])
    outs_ref, dx_ref, grads_ref = olora.lora_qkv_autograd(
        x.float().reshape(-1, K), list(refs.values()), [d.float().reshape(-1, d.shape[-1]) for d in douts])
    for out, ref in zip((Q, Kt, V), outs_ref):
        assert olora.max_rel_err(out.reshape(ref.shape), ref) < TOL
    assert olora.max_rel_err(xg.grad.reshape(-1, K), dx_ref) < TOL
    for name, (dA_ref, dB_ref) in zip(Ns, grads_ref):
        lin = getattr(attn, name)
        assert olora.max_rel_err(lin.lora_A["default"].weight.grad, dA_ref) < TOL
        assert olora.max_rel_err(lin.lora_B["default"].weight.grad, dB_ref) < TOL


@pytest.mark.parametrize("act_order,fwd_launches,bwd_launches", [(False, 1, 1), ("shared", 1, 1), (True, 3, 3)])
def test_qkv_launch_count(monkeypatch, act_order, fwd_launches, bwd_launches):
    """q, k, v go out as one fused-GEMM launch per direction unless their act-order permutations differ."""
    import fmsa_hip
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_qkv

    calls = {"fwd": 0, "bwd": 0}
    real_fwd, real_bwd = fmsa_hip.gptq_lora_fwd, fmsa_hip.gptq_lora_bwd_dx
    monkeypatch.setattr(fmsa_hip, "gptq_lora_fwd", lambda *a, **k: (calls.__setitem__("fwd", calls["fwd"] + 1), real_fwd(*a, **k))[1])
    monkeypatch.setattr(fmsa_hip, "gptq_lora_bwd_dx", lambda *a, **k: (calls.__setitem__("bwd", calls["bwd"] + 1), real_bwd(*a, **k))[1])
    attn = torch.nn.Module()
    for i, (name, N) in enumerate({"q_proj": 512, "k_proj": 128, "v_proj": 128}.items()):
        lin, *_ = make_lora_gptq_linear(512, N, 8, 16.0, seed=40 + i, act_order=act_order, device="cuda",
                                        order_seed=97 if act_order == "shared" else None)
        setattr(attn, name, lin)
    xg = randn((1, 64, 512), 5, torch.bfloat16).cuda().requires_grad_(True)
    Q, Kt, V = apply_lora_qkv(attn, xg)
    (Q.float().sum() + Kt.float().sum() + V.float().sum()).backward()
    assert calls == {"fwd": fwd_launches, "bwd": bwd_launches}


def _mlp(H, I, r, alpha, act_order, seed=20):
    mlp = torch.nn.Module()
    refs = {}
    for i, (name, (K, N)) in enumerate({"gate_proj": (H, I), "up_proj": (H, I), "down_proj": (I, H)}.items()):
        gs = 128 if K % 128 == 0 else 32
        lin, W, A, B = make_lora_gptq_linear(K, N, r, alpha, seed=seed + i, act_order=act_order, device="cuda", group_size=gs,
                                             order_seed=98 if act_order == "shared" else None)
        setattr(mlp, name, lin)
        refs[name] = (W, A, B, alpha / r)
    return mlp, refs


# two fixed shapes and six odd ones (H, I any multiple of 32: every tile cut in M, N, K; at least 33 tokens, fewer leave
# the 16-bit roundings of single products unaveraged and above the tolerance)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act_order", [False, True, "shared"])
@pytest.mark.parametrize("Bz,S,H,I", [(2, 128, 512, 1024), (1, 100, 256, 352), (1, 33, 96, 160), (3, 37, 160, 608),
                                      (1, 257, 672, 96), (2, 150, 32, 1312), (1, 513, 416, 288), (1, 64, 1184, 736)])
def test_lora_mlp(Bz, S, H, I, dtype, act_order):
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_mlp

    r, alpha = 16, 16.0
    mlp, refs = _mlp(H, I, r, alpha, act_order)
    x = randn((Bz, S, H), 2, dtype)
    dy = randn((Bz, S, H), 3, dtype)
    xg = x.cuda().requires_grad_(True)
    out = apply_lora_mlp(mlp, xg)
    out.backward(dy.cuda())
    ps = [(W, _q(A, dtype), _q(B, dtype), s) for W, A, B, s in (refs["gate_proj"], refs["up_proj"], refs["down_proj"])]
    out_ref, dx_ref, grads_ref, _ = olora.lora_mlp_autograd(x.float().reshape(-1, H), *ps, dy.float().reshape(-1, H))
    assert olora.max_rel_err(out.reshape(-1, H), out_ref) < TOL
    assert olora.max_rel_err(xg.grad.reshape(-1, H), dx_ref) < TOL
    for name, (dA_ref, dB_ref) in zip(("gate_proj", "up_proj", "down_proj"), grads_ref):
        lin = getattr(mlp, name)
        assert olora.max_rel_err(lin.lora_A["default"].weight.grad, dA_ref) < TOL, name
        assert olora.max_rel_err(lin.lora_B["default"].weight.grad, dB_ref) < TOL, name


@pytest.mark.parametrize("p", [0.1, 0.5])
def test_lora_w_dropout_mask(p):
    """A fixed Bernoulli mask as dropout: the LoRA branch sees x*mask, dX's LoRA part is masked
    by (x*mask != 0), and the adapter grads use x*mask."""
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_o_v2

    dtype, Bz, S, K, N, r, alpha = torch.bfloat16, 2, 64, 512, 512, 8, 1.0 * 8
    drop = MaskDropout(p, (Bz * S, K), seed=5)
    lin, W, A, B = make_lora_gptq_linear(K, N, r, alpha, seed=3, device="cuda", dropout=drop)
    x = randn((Bz, S, K), 2, dtype)
    dy = randn((Bz, S, N), 3, dtype)
    xg = x.cuda().requires_grad_(True)
    y = apply_lora_o_v2(lin, xg)
    y.backward(dy.cuda())
    x2 = x.float().reshape(-1, K)
    xd = x2 * drop.mask.cpu()
    s = alpha / r
    y_ref = olora.lora_linear(x2, W, _q(A, dtype), _q(B, dtype), s, xd=xd)
    dx_ref, dA_ref, dB_ref = olora.lora_w_manual(x2, W, _q(A, dtype), _q(B, dtype), s, dy.float().reshape(-1, N), xd=xd)
    assert olora.max_rel_err(y.reshape(-1, N), y_ref) < TOL
    assert olora.max_rel_err(xg.grad.reshape(-1, K), dx_ref) < TOL
    assert olora.max_rel_err(lin.lora_A["default"].weight.grad, dA_ref) < TOL
    assert olora.max_rel_err(lin.lora_B["default"].weight.grad, dB_ref) < TOL


def test_adapters_disabled_is_base_only():
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_o_v2

    dtype, K, N = torch.bfloat16, 512, 256
    lin, W, A, B = make_lora_gptq_linear(K, N, 8, 8.0, seed=3, device="cuda", bias=True)
    lin.enable_adapters(False)
    x = randn((1, 64, K), 2, dtype)
    xg = x.cuda().requires_grad_(True)
    y = apply_lora_o_v2(lin, xg)
    y.backward(torch.ones_like(y))
    ref = x.float().reshape(-1, K) @ W + lin.base_layer.bias.float().cpu()
    assert olora.max_rel_err(y.reshape(-1, N), ref) < TOL
    assert olora.max_rel_err(xg.grad.reshape(-1, K), torch.ones(64, N) @ W.t()) < TOL
    assert lin.lora_A["default"].weight.grad is None
