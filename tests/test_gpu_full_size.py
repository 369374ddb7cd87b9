"""Parity at the benchmark's full shapes.  The oracle cannot run the whole layer at these sizes in
seconds, so each case leans on properties that do not depend on size:
  * every output except dA / dB is row-wise in the tokens: a random subset of token rows of the
    full-size run is compared with the fp32 oracle (exact dequantisation of the complete weights,
    unfused graph differentiated by autograd) run on just those rows;
  * dA / dB are sums over tokens: the full run must equal the sum of the runs over the two halves
    of the tokens (each of which is covered by the row check again), and the row-subset run's
    dA / dB are compared with the oracle directly.
Tolerance: max |out - ref| / max |ref| <= 1e-2 per tensor (bf16 storage, fp32 accumulation)."""
import numpy as np
import pytest
import torch

from oracle import gptq as ogptq
from oracle import lora as olora
from oracle import nf4 as onf4

pytestmark = pytest.mark.gpu

TOL = 1e-2
DT = torch.bfloat16
N_ROWS = 96


def _gptq_lora(K, N, r, alpha, seed, act_order=False, group=128, order_seed=None):
    """LoraLinear(QuantLinear) quantised on the GPU; returns (module, fp32 dense W [K, N] on the CPU
    from the oracle's dequantisation of the packed buffers, A, B rounded to the activation dtype)."""
    from fms_acceleration_peft import LoraLinear
    from fms_acceleration_peft.quantizer import quantize_linear

    gen = torch.Generator(device="cuda").manual_seed(seed)
    W = torch.randn(N, K, generator=gen, device="cuda") * 0.02
    g_idx = None
    if act_order:
        perm = torch.randperm(K, generator=torch.Generator().manual_seed(seed + 4 if order_seed is None else order_seed))
        g_idx = (torch.arange(K) // group)[perm].to(torch.int32).cuda()
    ql = quantize_linear(W, group, g_idx=g_idx).cuda()
    del W
    lin = LoraLinear(ql, r, alpha).cuda()
    g2 = torch.Generator().manual_seed(seed + 1)
    lin.lora_B["default"].weight.data.copy_(torch.randn(N, r, generator=g2) * 0.02)
    dense = ogptq.dequant_torch(ql.qweight.cpu(), ql.scales.cpu(), ql.qzeros.cpu(), ql.g_idx.cpu())
    A = lin.lora_A["default"].weight.detach().cpu().to(DT).float()
    B = lin.lora_B["default"].weight.detach().cpu().to(DT).float()
    return lin, dense, A, B


def _nf4_lora(K, N, r, alpha, seed):
    from fms_acceleration_peft import Linear4bit, LoraLinear

    gen = torch.Generator(device="cuda").manual_seed(seed)
    W = torch.randn(N, K, generator=gen, device="cuda") * 0.02
    base = Linear4bit.from_dense(W, compute_dtype=DT)
    del W
    lin = LoraLinear(base, r, alpha).cuda()
    g2 = torch.Generator().manual_seed(seed + 1)
    lin.lora_B["default"].weight.data.copy_(torch.randn(N, r, generator=g2) * 0.02)
    qs = base.weight.quant_state
    q = {"packed": base.weight.data.cpu().numpy(), "absmax_q": qs.absmax.cpu().numpy(),
         "absmax2": qs.state2.absmax.cpu().numpy(), "code2": qs.state2.code.cpu().numpy(),
         "offset": np.float32(float(qs.offset)), "shape": (N, K), "blocksize": 64, "blocksize2": 256}
    assert np.array_equal(qs.code.cpu().numpy(), onf4.NF4)
    dense = onf4.dequant(q, "fp32").t().contiguous()
    A = lin.lora_A["default"].weight.detach().cpu().to(DT).float()
    B = lin.lora_B["default"].weight.detach().cpu().to(DT).float()
    return lin, dense, A, B


def _grads(mods):
    out = []
    for m in mods:
        out += [m.lora_A["default"].weight.grad.clone(), m.lora_B["default"].weight.grad.clone()]
    return out


def _zero(mods):
    for m in mods:
        m.lora_A["default"].weight.grad = None
        m.lora_B["default"].weight.grad = None


def _run(fn, mods, x, douts):
    """Forward + backward on the GPU; returns (outs, dx, [dA, dB, ...])."""
    _zero(mods)
    xg = x.clone().requires_grad_(True)
    outs = fn(xg)
    outs = outs if isinstance(outs, tuple) else (outs,)
    torch.autograd.backward(list(outs), list(douts))
    return [o.detach() for o in outs], xg.grad, _grads(mods)


def _check_split_sum(fn, mods, x, douts, full_grads):
    h = x.shape[0] // 2
    _, _, g1 = _run(fn, mods, x[:h], [d[:h] for d in douts])
    _, _, g2 = _run(fn, mods, x[h:], [d[h:] for d in douts])
    for gf, a, b in zip(full_grads, g1, g2):
        assert olora.max_rel_err(gf.float().cpu(), (a.float() + b.float()).cpu()) < 2e-3


def _rows(M, seed):
    return torch.randperm(M, generator=torch.Generator().manual_seed(seed))[:N_ROWS].sort().values


def _mlp_case(make, M, H, I, r, alpha, act_order=False):
    kw = {"act_order": act_order} if make is _gptq_lora else {}
    mlp = torch.nn.Module()
    ps = []
    for i, (name, K, N) in enumerate((("gate_proj", H, I), ("up_proj", H, I), ("down_proj", I, H))):
        lin, W, A, B = make(K, N, r, alpha, seed=20 + 10 * i, **kw)
        setattr(mlp, name, lin)
        ps.append((W, A, B, alpha / r))
    mods = [mlp.gate_proj, mlp.up_proj, mlp.down_proj]
    if make is _gptq_lora:
        from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_mlp as op
    else:
        from fms_acceleration_foak.fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_mlp_swiglu as op
    fn = lambda t: op(mlp, t)  # noqa: E731
    gen = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn(M, H, generator=gen, device="cuda").to(DT)
    dy = torch.randn(M, H, generator=gen, device="cuda").to(DT)
    (out,), dx, grads = _run(fn, mods, x, [dy])
    rows = _rows(M, 7)
    # the row-subset run on the GPU gives dA / dB of exactly the rows the oracle sees
    (out_s,), dx_s, grads_s = _run(fn, mods, x[rows.cuda()].contiguous(), [dy[rows.cuda()].contiguous()])
    out_ref, dx_ref, grads_ref, _ = olora.lora_mlp_autograd(x[rows.cuda()].float().cpu(), *ps, dy[rows.cuda()].float().cpu())
    assert olora.max_rel_err(out[rows.cuda()].cpu(), out_ref) < TOL
    assert olora.max_rel_err(dx[rows.cuda()].cpu(), dx_ref) < TOL
    assert olora.max_rel_err(out_s.cpu(), out_ref) < TOL and olora.max_rel_err(dx_s.cpu(), dx_ref) < TOL
    flat_ref = [t for pair in grads_ref for t in pair]
    for got, ref in zip(grads_s, flat_ref):
        assert olora.max_rel_err(got.cpu(), ref) < 2 * TOL
    _check_split_sum(fn, mods, x, [dy], grads)


def test_config2_llama3_8b_mlp():
    _mlp_case(_gptq_lora, 8192, 4096, 14336, 16, 16.0)


def test_config4_llama2_70b_mlp_act_order_r64():
    _mlp_case(_gptq_lora, 4096, 8192, 28672, 64, 128.0, act_order=True)


def test_config5_mistral_7b_mlp_nf4_r8():
    _mlp_case(_nf4_lora, 16384, 4096, 14336, 8, 16.0)


def test_config3_llama3_8b_qkvo():
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_o_v2, apply_lora_qkv

    M, H, r, alpha = 8192, 4096, 16, 32.0
    attn = torch.nn.Module()
    projs = []
    for i, (name, N) in enumerate((("q_proj", 4096), ("k_proj", 1024), ("v_proj", 1024))):
        lin, W, A, B = _gptq_lora(H, N, r, alpha, seed=50 + 10 * i)
        setattr(attn, name, lin)
        projs.append((W, A, B, alpha / r))
    mods = [attn.q_proj, attn.k_proj, attn.v_proj]
    gen = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn(M, H, generator=gen, device="cuda").to(DT)
    douts = [torch.randn(M, n, generator=gen, device="cuda").to(DT) for n in (4096, 1024, 1024)]
    fn = lambda t: apply_lora_qkv(attn, t)  # noqa: E731
    outs, dx, grads = _run(fn, mods, x, douts)
    rows = _rows(M, 8).cuda()
    outs_s, dx_s, grads_s = _run(fn, mods, x[rows].contiguous(), [d[rows].contiguous() for d in douts])
    outs_ref, dx_ref, grads_ref = olora.lora_qkv_autograd(x[rows].float().cpu(), projs, [d[rows].float().cpu() for d in douts])
    for o, o_ref in zip(outs, outs_ref):
        assert olora.max_rel_err(o[rows].cpu(), o_ref) < TOL
    assert olora.max_rel_err(dx[rows].cpu(), dx_ref) < TOL
    for got, ref in zip(grads_s, [t for pair in grads_ref for t in pair]):
        assert olora.max_rel_err(got.cpu(), ref) < 2 * TOL
    _check_split_sum(fn, mods, x, douts, grads)

    # o_proj
    lin, W, A, B = _gptq_lora(H, H, r, alpha, seed=90)
    fo = lambda t: apply_lora_o_v2(lin, t)  # noqa: E731
    dO = torch.randn(M, H, generator=gen, device="cuda").to(DT)
    (o,), dxo, g = _run(fo, [lin], x, [dO])
    (o_s,), _, g_s = _run(fo, [lin], x[rows].contiguous(), [dO[rows].contiguous()])
    y_ref, dxo_ref, dA_ref, dB_ref = olora.lora_w_autograd(x[rows].float().cpu(), W, A, B, alpha / r, dO[rows].float().cpu())
    assert olora.max_rel_err(o[rows].cpu(), y_ref) < TOL
    assert olora.max_rel_err(dxo[rows].cpu(), dxo_ref) < TOL
    assert olora.max_rel_err(g_s[0].cpu(), dA_ref) < 2 * TOL and olora.max_rel_err(g_s[1].cpu(), dB_ref) < 2 * TOL
    _check_split_sum(fo, [lin], x, [dO], g)


@pytest.fixture
def float16(monkeypatch):
    """The reference's own arithmetic for this path (fp16 dequantisation output, fp16 benchmark runs): the same
    cases with fp16 activations, which take the packed-half unpack kernels."""
    import sys

    monkeypatch.setattr(sys.modules[__name__], "DT", torch.float16)


def test_config2_llama3_8b_mlp_float16(float16):
    _mlp_case(_gptq_lora, 8192, 4096, 14336, 16, 16.0)


def test_config3_llama3_8b_qkvo_float16(float16):
    test_config3_llama3_8b_qkvo()


def test_no_worse_than_materialised_decomposition():
    """The fused kernels' error against the fp32 oracle is no worse than that of the decomposition
    the reference runs (dense weight rounded to the activation dtype, library matmul, separate LoRA
    matmuls each rounded) executed on the same GPU."""
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_o_v2

    M, H, r, alpha = 8192, 4096, 16, 32.0
    s = alpha / r
    lin, W, A, B = _gptq_lora(H, H, r, alpha, seed=90)
    gen = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn(M, H, generator=gen, device="cuda").to(DT)
    dO = torch.randn(M, H, generator=gen, device="cuda").to(DT)
    (o,), dx, _ = _run(lambda t: apply_lora_o_v2(lin, t), [lin], x, [dO])
    rows = _rows(M, 9).cuda()
    y_ref, dx_ref, _, _ = olora.lora_w_autograd(x[rows].float().cpu(), W, A, B, s, dO[rows].float().cpu())
    Wd = lin.base_layer.dequantize(DT) if hasattr(lin.base_layer, "dequantize") else W.cuda().to(DT)
    Ad, Bd = A.cuda().to(DT), B.cuda().to(DT)
    xs, ds = x[rows], dO[rows]
    y_dec = xs @ Wd + (xs @ Ad.t()) @ (s * Bd.t())
    dx_dec = ds @ Wd.t() + (ds @ Bd) @ (s * Ad)
    for mine, dec, ref in ((o[rows], y_dec, y_ref), (dx[rows], dx_dec, dx_ref)):
        e_mine, e_dec = olora.max_rel_err(mine.cpu(), ref), olora.max_rel_err(dec.cpu(), ref)
        assert e_mine < TOL and e_mine <= 1.25 * e_dec + 1e-4, (e_mine, e_dec)
        # the element-wise figure (entries above 1 % of the tensor's maximum): the mean must be no worse than the
        # decomposition's either, and the worst single entry (an entry just above the floor, a 16-bit rounding step
        # away from its value) stays within twice the decomposition's worst
        (m_mine, a_mine), (m_dec, a_dec) = olora.elementwise_rel_err(mine, ref, 1e-2), olora.elementwise_rel_err(dec, ref, 1e-2)
        assert a_mine <= 1.25 * a_dec + 1e-5, (a_mine, a_dec)
        assert m_mine <= 2.0 * m_dec + 1e-3, (m_mine, m_dec)
