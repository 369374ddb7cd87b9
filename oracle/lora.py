"""Unfused quantised-LoRA forward/backward on the CPU (torch), two independent statements.

(1) ``*_autograd``: the graph the reference's own parity test treats as ground truth -- the
    UNPATCHED module: dense dequantised W, ``x @ W``, PEFT-style ``lora_B(lora_A(dropout(x))) *
    scaling``, HF ``down(silu(gate(x)) * up(x))`` -- differentiated by torch.autograd
    (plugins/fused-ops-and-kernels/tests/test_fused_ops.py:400-438; unfused forward:
    GQ/nn_modules/triton_utils/dequant.py:132-161).
(2) ``*_manual``: the hand-derived backward formulas of the fused autograd functions
    (UL/gptq/fast_lora.py:822-831 LoRA_W, :591-711 LoRA_QKV, :351-398 LoRA_MLP, with the
    down-projection mask taken on h as for every other projection instead of the shape-mismatched
    in-place mask of :354-357, which cannot run for hidden != intermediate).

Everything is dtype-generic: run it in float64 to pin the math, in float32 as the tolerance
oracle for the GPU kernels.  W is [K, N] (input-major, as dequant248 returns it), A is
lora_A.weight [r, K], B is lora_B.weight [N, r].
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


# ---- single projection ---------------------------------------------------------------------------
def lora_linear(x, W, A, B, s, bias=None, xd=None):
    """y = x W + s (xd A^T) B^T (+ bias); xd = dropout(x), default x
    (matmul_lora, UL/gptq/fast_lora.py:143-169)."""
    y = x @ W
    if A is not None:
        xd = x if xd is None else xd
        y = y + (xd @ A.t()) @ (s * B.t())
    if bias is not None:
        y = y + bias
    return y


def lora_w_autograd(x, W, A, B, s, dy, bias=None):
    """Returns (y, dx, dA, dB) of LoRA_W via autograd; W is frozen."""
    x = x.detach().clone().requires_grad_(True)
    A = A.detach().clone().requires_grad_(True)
    B = B.detach().clone().requires_grad_(True)
    y = lora_linear(x, W, A, B, s, bias)
    y.backward(dy)
    return y.detach(), x.grad, A.grad, B.grad


def lora_w_manual(x, W, A, B, s, dy, xd=None):
    """dx, dA, dB by the closed forms (UL/gptq/fast_lora.py:822-831):
         T = dY B,  U = Xd A^T,  dA = s T^T Xd,  dB = s dY^T U,
         dX = dY W^T + (Xd != 0) * (T (s A))."""
    xd = x if xd is None else xd
    T = dy @ B
    U = xd @ A.t()
    dA = s * (T.t() @ xd)
    dB = s * (dy.t() @ U)
    dx = dy @ W.t() + (xd != 0).to(x.dtype) * (T @ (s * A))
    return dx, dA, dB


# ---- q, k, v sharing x ---------------------------------------------------------------------------
def lora_qkv_autograd(x, projs, douts):
    """projs: list of (W, A, B, s); douts: matching upstream grads. Returns (outs, dx, [(dA, dB)])."""
    x = x.detach().clone().requires_grad_(True)
    leaves = [(A.detach().clone().requires_grad_(True), B.detach().clone().requires_grad_(True)) for _, A, B, _ in projs]
    outs = [lora_linear(x, W, a, b, s) for (W, _, _, s), (a, b) in zip(projs, leaves)]
    torch.autograd.backward(outs, douts)
    return [o.detach() for o in outs], x.grad, [(a.grad, b.grad) for a, b in leaves]


def lora_qkv_manual(x, projs, douts):
    dx = torch.zeros_like(x)
    grads = []
    for (W, A, B, s), dy in zip(projs, douts):
        dxi, dA, dB = lora_w_manual(x, W, A, B, s, dy)
        dx = dx + dxi
        grads.append((dA, dB))
    return dx, grads


# ---- SwiGLU --------------------------------------------------------------------------------------
def swiglu_fwd(e, g):
    """h = silu(e) * g with the rounding points of UL/swiglu.py:26-33: silu in fp32, rounded to the
    storage dtype, product in the storage dtype."""
    e32 = e.float()
    f = (e32 * torch.sigmoid(e32)).to(g.dtype)
    return f * g


def swiglu_bwd(dh, e, g):
    """(h, d_g, d_e) with the rounding points of UL/swiglu.py:65-83 (the reference names d_g
    'df' and d_e 'de')."""
    e32 = e.float()
    se = torch.sigmoid(e32)
    f = (se * e32).to(dh.dtype)
    h = f * g
    d_g = dh * f
    dg = dh * g
    d_e = (dg.float() * se * (1.0 + e32 * (1.0 - se))).to(dh.dtype)
    return h, d_g, d_e


# ---- MLP -----------------------------------------------------------------------------------------
def lora_mlp_forward(x, gate, up, down):
    """gate/up/down = (W, A, B, s).  Returns (out, e, g, h)."""
    e = lora_linear(x, *gate)
    g = lora_linear(x, *up)
    h = F.silu(e) * g
    return lora_linear(h, *down), e, g, h


def lora_mlp_autograd(x, gate, up, down, dy):
    x = x.detach().clone().requires_grad_(True)
    leaves = []
    ps = []
    for W, A, B, s in (gate, up, down):
        a = A.detach().clone().requires_grad_(True)
        b = B.detach().clone().requires_grad_(True)
        leaves.append((a, b))
        ps.append((W, a, b, s))
    out, e, g, h = lora_mlp_forward(x, *ps)
    out.backward(dy)
    return out.detach(), x.grad, [(a.grad, b.grad) for a, b in leaves], (e.detach(), g.detach(), h.detach())


def lora_mlp_manual(x, gate, up, down, dy):
    """Closed-form backward of LoRA_MLP (UL/gptq/fast_lora.py:351-398), in the dtype of x with no
    intermediate rounding (the rounding points are exercised separately by swiglu_bwd)."""
    Wg, Ag, Bg, sg = gate
    Wu, Au, Bu, su = up
    Wd, Ad, Bd, sd = down
    e = lora_linear(x, *gate)
    g = lora_linear(x, *up)
    se = torch.sigmoid(e)
    f = se * e
    h = f * g
    # down projection: dh = dY Wd^T + (h != 0) * (dY Bd)(sd Ad)
    Td = dy @ Bd
    dh = dy @ Wd.t() + (h != 0).to(x.dtype) * (Td @ (sd * Ad))
    d_g = dh * f
    d_e = dh * g * se * (1.0 + e * (1.0 - se))
    dAd = sd * (Td.t() @ h)
    dBd = sd * (dy.t() @ (h @ Ad.t()))
    dxu, dAu, dBu = lora_w_manual(x, Wu, Au, Bu, su, d_g)
    dxg, dAg, dBg = lora_w_manual(x, Wg, Ag, Bg, sg, d_e)
    return dxu + dxg, [(dAg, dBg), (dAu, dBu), (dAd, dBd)]


# ---- seeded inputs -------------------------------------------------------------------------------
def make_lora(K, N, r, seed, dtype=torch.float32):
    """A kaiming-uniform(a=sqrt(5)) [r, K] (PEFT's default), B ~ N(0, 0.02) [N, r] (non-zero so that
    gradients are non-trivial, as test_fused_ops.py:387-389 re-initialises lora_B)."""
    gen = torch.Generator().manual_seed(seed)
    bound = 1.0 / (K ** 0.5)  # kaiming_uniform_(a=sqrt(5)) on [r, K]: gain*sqrt(3/fan_in) = 1/sqrt(K)
    A = (torch.rand(r, K, generator=gen, dtype=torch.float32) * 2 - 1) * bound
    B = torch.randn(N, r, generator=gen, dtype=torch.float32) * 0.02
    return A.to(dtype), B.to(dtype)


def max_rel_err(out, ref):
    """max |out - ref| / max |ref| (per tensor): the tolerance metric used for the GPU kernels."""
    out = out.detach().double().cpu()
    ref = ref.detach().double().cpu()
    return ((out - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()


def elementwise_rel_err(out, ref, floor=1e-2):
    """(max, mean) of |out - ref| / |ref| over the entries with |ref| > floor * max |ref|: the element-wise
    figure reported next to max_rel_err (entries near zero are left out, where a relative error says nothing)."""
    out = out.detach().double().cpu()
    ref = ref.detach().double().cpu()
    keep = ref.abs() > floor * ref.abs().max()
    if not bool(keep.any()):
        return 0.0, 0.0
    rel = (out[keep] - ref[keep]).abs() / ref[keep].abs()
    return rel.max().item(), rel.mean().item()
