"""Pins the oracle's forward/backward math: torch.autograd of the unfused graph against the
hand-derived closed forms (fp64), finite differences, and special cases."""
import pytest
import torch

from oracle import lora as olora
from tests.helpers import make_gptq, randn

D = torch.float64


def _case(M=16, K=64, N=32, r=8, seed=0):
    w = make_gptq(K, N, 32, seed=seed)
    A, B = olora.make_lora(K, N, r, seed + 1, D)
    return w["dense"].to(D), A, B, randn((M, K), seed + 2, D), randn((M, N), seed + 3, D)


def test_lora_w_autograd_equals_closed_form():
    W, A, B, x, dy = _case()
    y, dx, dA, dB = olora.lora_w_autograd(x, W, A, B, 2.0, dy)
    dx2, dA2, dB2 = olora.lora_w_manual(x, W, A, B, 2.0, dy)
    for a, b in ((dx, dx2), (dA, dA2), (dB, dB2)):
        torch.testing.assert_close(a, b, rtol=1e-12, atol=1e-12)
    assert dA.shape == A.shape and dB.shape == B.shape


def test_lora_w_finite_differences():
    W, A, B, x, dy = _case(M=4, K=32, N=32, r=8)
    s = 0.5
    loss = lambda xx, aa, bb: (olora.lora_linear(xx, W, aa, bb, s) * dy).sum()  # noqa: E731
    _, dx, dA, dB = olora.lora_w_autograd(x, W, A, B, s, dy)
    eps = 1e-6
    for tensor, grad, idx in ((x, dx, (1, 3)), (A, dA, (2, 5)), (B, dB, (7, 1))):
        t = tensor.clone()
        t[idx] += eps
        args = [x, A, B]
        args[[id(a) for a in args].index(id(tensor))] = t
        num = (loss(*args) - loss(x, A, B)) / eps
        assert abs(num.item() - grad[idx].item()) < 1e-5 * max(1.0, abs(grad[idx].item()))


def test_special_cases():
    W, A, B, x, dy = _case()
    # B = 0: output is the base GEMM and dA vanishes
    y, dx, dA, dB = olora.lora_w_autograd(x, W, A, torch.zeros_like(B), 2.0, dy)
    torch.testing.assert_close(y, x @ W)
    assert dA.abs().max() == 0 and dB.abs().max() > 0
    # A = 0: dB vanishes
    _, _, dA, dB = olora.lora_w_autograd(x, W, torch.zeros_like(A), B, 2.0, dy)
    assert dB.abs().max() == 0 and dA.abs().max() > 0
    # the LoRA contribution is linear in s
    y1 = olora.lora_linear(x, W, A, B, 1.0) - x @ W
    y3 = olora.lora_linear(x, W, A, B, 3.0) - x @ W
    torch.testing.assert_close(y3, 3 * y1)
    # adapters disabled: base only
    torch.testing.assert_close(olora.lora_linear(x, W, None, None, None), x @ W)


def test_zero_inputs_mask_the_lora_part_of_dx():
    """dX's LoRA term carries the factor (Xd != 0): exact zeros in the (post-dropout) input switch it
    off.  autograd of the unfused graph has no such factor, so the two agree only away from zeros."""
    W, A, B, x, dy = _case()
    x[::3, ::2] = 0
    _, dx_auto, _, _ = olora.lora_w_autograd(x, W, A, B, 2.0, dy)
    dx_man, _, _ = olora.lora_w_manual(x, W, A, B, 2.0, dy)
    nz = x != 0
    torch.testing.assert_close(dx_man[nz], dx_auto[nz])
    torch.testing.assert_close(dx_man[~nz], (dy @ W.t())[~nz])


def test_qkv_autograd_equals_closed_form():
    K, r, M = 64, 8, 12
    x = randn((M, K), 1, D)
    projs, douts = [], []
    for i, N in enumerate((64, 32, 32)):
        w = make_gptq(K, N, 32, seed=10 + i)
        A, B = olora.make_lora(K, N, r, 20 + i, D)
        projs.append((w["dense"].to(D), A, B, 2.0))
        douts.append(randn((M, N), 30 + i, D))
    _, dx, grads = olora.lora_qkv_autograd(x, projs, douts)
    dx2, grads2 = olora.lora_qkv_manual(x, projs, douts)
    torch.testing.assert_close(dx, dx2, rtol=1e-12, atol=1e-12)
    for (a, b), (a2, b2) in zip(grads, grads2):
        torch.testing.assert_close(a, a2, rtol=1e-12, atol=1e-12)
        torch.testing.assert_close(b, b2, rtol=1e-12, atol=1e-12)


def test_mlp_autograd_equals_closed_form():
    """LoRA_MLP backward formulas (with the down-projection mask taken on h) against autograd of
    down(silu(gate(x)) * up(x))."""
    H, I, r, M = 64, 96, 8, 10
    x = randn((M, H), 1, D)
    dy = randn((M, H), 2, D)
    ps = []
    for i, (K, N) in enumerate(((H, I), (H, I), (I, H))):
        w = make_gptq(K, N, 32, seed=40 + i)
        A, B = olora.make_lora(K, N, r, 50 + i, D)
        ps.append((w["dense"].to(D), A, B, 1.5))
    out, dx, grads, _ = olora.lora_mlp_autograd(x, *ps, dy)
    dx2, grads2 = olora.lora_mlp_manual(x, *ps, dy)
    torch.testing.assert_close(dx, dx2, rtol=1e-10, atol=1e-10)
    for (a, b), (a2, b2) in zip(grads, grads2):
        torch.testing.assert_close(a, a2, rtol=1e-10, atol=1e-10)
        torch.testing.assert_close(b, b2, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_swiglu_rounding_points_against_silu(dtype):
    e, g, dh = randn((64, 96), 1, dtype), randn((64, 96), 2, dtype), randn((64, 96), 3, dtype)
    tol = 2 ** -7 if dtype == torch.bfloat16 else 2 ** -10
    h = olora.swiglu_fwd(e, g)
    ref = torch.nn.functional.silu(e.float()) * g.float()
    assert olora.max_rel_err(h.float(), ref) < 2 * tol
    # backward against autograd of silu(e) * g in fp64
    e64 = e.double().requires_grad_(True)
    g64 = g.double().requires_grad_(True)
    (torch.nn.functional.silu(e64) * g64).backward(dh.double())
    h2, d_g, d_e = olora.swiglu_bwd(dh, e, g)
    assert torch.equal(h2, h)
    assert olora.max_rel_err(d_g.float(), g64.grad) < 4 * tol
    assert olora.max_rel_err(d_e.float(), e64.grad) < 4 * tol


def test_config1_plumbing_on_cpu():
    """BASELINE config 1: one GPTQ-LoRA linear through the unfused path on the CPU -- x [512, 2048],
    W [2048, 2048] RTN group 128, rank 16, alpha 16 -- autograd equals the closed forms in fp32."""
    M, K, N, r = 512, 2048, 2048, 16
    w = make_gptq(K, N, 128, seed=0)
    A, B = olora.make_lora(K, N, r, 1)
    x, dy = randn((M, K), 2), randn((M, N), 3)
    y, dx, dA, dB = olora.lora_w_autograd(x, w["dense"], A, B, 1.0, dy)
    dx2, dA2, dB2 = olora.lora_w_manual(x, w["dense"], A, B, 1.0, dy)
    assert y.shape == (M, N)
    for a, b in ((dx, dx2), (dA, dA2), (dB, dB2)):
        assert olora.max_rel_err(a, b) < 1e-5


def test_error_metrics_known_answers():
    """max_rel_err is relative to the largest reference entry; elementwise_rel_err leaves out entries below
    the floor (1e-2 of the largest) and returns (max, mean) of the per-entry relative errors of the rest."""
    ref = torch.tensor([1.0, 2.0, 0.001, -4.0])
    out = torch.tensor([1.1, 2.0, 0.002, -4.0])
    assert abs(olora.max_rel_err(out, ref) - 0.1 / 4.0) < 1e-6
    mx, mean = olora.elementwise_rel_err(out, ref, 1e-2)
    assert abs(mx - 0.1) < 1e-6 and abs(mean - 0.1 / 3) < 1e-6   # the 0.001 entry (100 % off) is below the floor
    mx_all, _ = olora.elementwise_rel_err(out, ref, 0.0)
    assert abs(mx_all - 1.0) < 1e-6
    assert olora.elementwise_rel_err(torch.zeros(3), torch.zeros(3)) == (0.0, 0.0)
