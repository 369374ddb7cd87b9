"""The HIP kernels (through the C ABI and the drop-in operators) against the committed vectors of
tests/golden/hot_path_small.npz.  Bit-exact where the expected value is one rounding of an exact
product (GPTQ and NF4 dequantisation); 1e-2 of the largest reference entry for the GEMM paths (bf16
inputs, fp32 accumulation), the tolerance of the fused-op tests; the SwiGLU and norm / rotary kernels
use hardware exp2 / rcp / rsq, so their 16-bit results may differ from the vectors in the last place."""
import os

import numpy as np
import pytest
import torch

from oracle import lora as olora

pytestmark = pytest.mark.gpu
FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hot_path_small.npz")
TOL = 1e-2


@pytest.fixture(scope="module")
def gold():
    with np.load(FIXTURE) as z:
        return {k: z[k] for k in z.files}


def _t16(bits, dtype=torch.bfloat16):
    return torch.from_numpy(bits.view(np.int16).copy()).view(dtype)


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _lora_linear(gold, prefix, r, alpha, K, N):
    from fms_acceleration_peft import LoraLinear, QuantLinear

    ql = QuantLinear(4, 64, K, N, False)
    ql.load_packed(*(gold[f"{prefix}.{k}"] for k in ("qweight", "qzeros", "scales", "g_idx")))
    lin = LoraLinear(ql, r, alpha, dtype=torch.float32)
    lin.lora_A["default"].weight.data.copy_(_t16(gold[f"{prefix}.A"]).float())
    lin.lora_B["default"].weight.data.copy_(_t16(gold[f"{prefix}.B"]).float())
    return lin.cuda()


@pytest.mark.parametrize("tag", ["deq", "deq_act"])
def test_dequant_bit_exact(gold, tag):
    import fmsa_hip

    qw, qz, sc, gi = (_dev(gold[f"{tag}.{k}"]) for k in ("qweight", "qzeros", "scales", "g_idx"))
    for name, dtype in (("W_fp16", torch.float16), ("W_bf16", torch.bfloat16)):
        W = fmsa_hip.gptq_dequant(qw, sc, qz, gi, 64, 0, dtype)
        assert torch.equal(W.cpu(), _t16(gold[f"{tag}.{name}"], dtype))
    if tag == "deq":  # the same weights from v1 zero points
        W = fmsa_hip.gptq_dequant(qw, sc, _dev(gold["deq.qzeros_v1"]), gi, 64, 1, torch.bfloat16)
        assert torch.equal(W.cpu(), _t16(gold["deq.W_bf16"]))


def test_nf4_dequant_bit_exact(gold):
    import fmsa_hip
    from oracle import nf4 as onf4

    shape = tuple(int(v) for v in gold["nf4.shape"])
    for name, dtype in (("W_bf16", torch.bfloat16), ("W_fp16", torch.float16)):
        W = fmsa_hip.nf4_dequant(_dev(gold["nf4.packed"]), _dev(gold["nf4.absmax_q"]), _dev(gold["nf4.absmax2"]), _dev(gold["nf4.code2"]),
                                 _dev(onf4.NF4), float(gold["nf4.offset"]), shape, int(gold["nf4.blocksize"]),
                                 int(gold["nf4.blocksize2"]), dtype)
        assert torch.equal(W.cpu(), _t16(gold[f"nf4.{name}"], dtype))
    # the same values through the one-time re-layout the fused kernels read
    qw, bs = fmsa_hip.nf4_prepare(_dev(gold["nf4.packed"]), _dev(gold["nf4.absmax_q"]), _dev(gold["nf4.absmax2"]), _dev(gold["nf4.code2"]),
                                  float(gold["nf4.offset"]), shape, int(gold["nf4.blocksize"]), int(gold["nf4.blocksize2"]))
    code = _dev(onf4.NF4)
    Wt = fmsa_hip.weight_dequant(fmsa_hip.make_codebook_weight(qw, code, bs, int(gold["nf4.blocksize"])), qw.device, torch.bfloat16)
    assert torch.equal(Wt.t().contiguous().cpu(), _t16(gold["nf4.W_bf16"]))


def test_lora_w_vectors(gold):
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_o_v2

    s = float(gold["lora_w.s"])
    lin = _lora_linear(gold, "lora_w", 16, 16 * s, 256, 64)
    x = _t16(gold["lora_w.x"]).cuda().requires_grad_(True)
    y = apply_lora_o_v2(lin, x)
    y.backward(_t16(gold["lora_w.dy"]).cuda())
    for got, name in ((y, "y"), (x.grad, "dx"), (lin.lora_A["default"].weight.grad, "dA"), (lin.lora_B["default"].weight.grad, "dB")):
        assert olora.max_rel_err(got.detach().cpu(), torch.from_numpy(gold[f"lora_w.{name}"])) < TOL, name


def test_lora_mlp_vectors(gold):
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_mlp

    s = float(gold["mlp.s"])
    mlp = torch.nn.Module()
    for name, (K, N) in (("gate", (256, 128)), ("up", (256, 128)), ("down", (128, 256))):
        setattr(mlp, f"{name}_proj", _lora_linear(gold, f"mlp.{name}", 8, 8 * s, K, N))
    x = _t16(gold["mlp.x"]).cuda().requires_grad_(True)
    out = apply_lora_mlp(mlp, x)
    out.backward(_t16(gold["mlp.dy"]).cuda())
    assert olora.max_rel_err(out.detach().cpu(), torch.from_numpy(gold["mlp.out"])) < TOL
    assert olora.max_rel_err(x.grad.cpu(), torch.from_numpy(gold["mlp.dx"])) < TOL
    for name in ("gate", "up", "down"):
        lin = getattr(mlp, f"{name}_proj")
        assert olora.max_rel_err(lin.lora_A["default"].weight.grad.cpu(), torch.from_numpy(gold[f"mlp.{name}.dA"])) < TOL, name
        assert olora.max_rel_err(lin.lora_B["default"].weight.grad.cpu(), torch.from_numpy(gold[f"mlp.{name}.dB"])) < TOL, name


def _close_16bit(got, want_bits, dtype, frac=0.98):
    """Equal on at least `frac` of the entries and never more than one step of the 16-bit format apart."""
    want = _t16(want_bits, dtype)
    ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
    g, w = got.cpu().float(), want.float()
    return (g == w).float().mean().item() >= frac and bool(torch.all((g - w).abs() <= w.abs() * ulp + 1e-30))


@pytest.mark.parametrize("tag,dtype", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_swiglu_vectors(gold, tag, dtype):
    import fmsa_hip

    e, g, dh = (_t16(gold[f"swiglu.{tag}.{k}"], dtype).cuda() for k in ("e", "g", "dh"))
    assert _close_16bit(fmsa_hip.swiglu_fwd(e, g), gold[f"swiglu.{tag}.h"], dtype)
    e2, g2 = e.clone(), g.clone()
    h = fmsa_hip.swiglu_bwd(dh, e2, g2)  # in place: e <- d_g, g <- d_e
    assert _close_16bit(h, gold[f"swiglu.{tag}.h"], dtype)
    assert _close_16bit(e2, gold[f"swiglu.{tag}.d_g"], dtype)
    assert _close_16bit(g2, gold[f"swiglu.{tag}.d_e"], dtype, frac=0.95)


def test_norm_rope_cross_entropy_vectors(gold):
    import fmsa_hip

    x, w, dy = (_t16(gold[f"rms.{k}"]).cuda() for k in ("x", "w", "dy"))
    y, r = fmsa_hip.rms_layernorm_fwd(x, w, 1e-5)
    assert _close_16bit(y, gold["rms.y"], torch.bfloat16) and torch.allclose(r.cpu(), torch.from_numpy(gold["rms.r"]), rtol=1e-5)
    dx = fmsa_hip.rms_layernorm_bwd(dy.clone(), x, w, r)
    assert olora.max_rel_err(dx.cpu(), _t16(gold["rms.dx"]).float()) < 2.0 ** -7
    cos, sin = _dev(gold["rope.cos"]), _dev(gold["rope.sin"])
    for name, backward in (("fwd", False), ("bwd", True)):
        q = fmsa_hip.rope_embedding_(_t16(gold["rope.q"]).cuda(), cos, sin, 2, 64, backward)
        assert _close_16bit(q, gold[f"rope.{name}"], torch.bfloat16)
    logits, labels = _dev(gold["ce.logits"]), _dev(gold["ce.labels"])
    loss, lse = fmsa_hip.cross_entropy_fwd(logits, labels)
    assert torch.allclose(loss.cpu(), torch.from_numpy(gold["ce.loss"]), rtol=2e-5, atol=2e-5)
    assert torch.allclose(lse.cpu(), torch.from_numpy(gold["ce.lse"]), rtol=2e-5, atol=2e-5)
    grad = fmsa_hip.cross_entropy_bwd_(logits.clone(), _dev(gold["ce.dloss"]), lse, labels)
    assert torch.allclose(grad.cpu(), torch.from_numpy(gold["ce.grad"]), atol=2e-5)
    fl, fg = fmsa_hip.cross_entropy_fused_(logits.clone(), labels, torch.tensor([0.2], device="cuda"), 0.1)
    assert torch.allclose(fl.double().cpu(), torch.from_numpy(gold["ce.fused_loss"]), rtol=2e-5, atol=2e-5)
    assert torch.allclose(fg.double().cpu(), torch.from_numpy(gold["ce.fused_grad"]), atol=1e-5)
