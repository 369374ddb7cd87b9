"""RMS layer norm and rotary embedding kernels (through the C ABI) against the CPU oracle, and the
drop-in operators against transformers' own modules.  Floating-point kernels: the tolerance is one
rounding of the storage type (bf16 2^-7, fp16 2^-10 relative to the tensor's scale; fp32 1e-5) --
the kernels use the hardware rsqrt and a single final rounding."""
import pytest
import torch

from oracle import norm_rope as onr
from tests.helpers import randn

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 1e-5}


def _close(a, b, dtype):
    a, b = a.float().cpu(), b.float().cpu()
    return (a - b).abs().max().item() <= TOL[dtype] * max(b.abs().max().item(), 1e-6)


@pytest.mark.parametrize("gemma", [False, True])
@pytest.mark.parametrize("xdt,wdt", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
                                      (torch.float32, torch.float32), (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("M,C", [(37, 4096), (5, 520), (300, 1024)])
def test_rms_layernorm(M, C, xdt, wdt, gemma):
    import fmsa_hip

    x = randn((M, C), 1, xdt, scale=2.0)
    w = (randn((C,), 2) * 0.5 + 1.0).to(wdt)
    dy = randn((M, C), 3, xdt)
    y, r = fmsa_hip.rms_layernorm_fwd(x.cuda(), w.cuda(), 1e-5, gemma)
    y_ref, r_ref = onr.rms_fwd(x, w, 1e-5, gemma)
    assert y.dtype == xdt and _close(y, y_ref, xdt)
    assert torch.allclose(r.cpu(), r_ref, rtol=1e-5)
    dyd = dy.cuda().clone()
    dx = fmsa_hip.rms_layernorm_bwd(dyd, x.cuda(), w.cuda(), r, gemma)
    assert dx.data_ptr() == dyd.data_ptr()  # written over dY
    assert _close(dx, onr.rms_bwd(dy, x, w, r_ref, gemma), xdt)


def _cos_sin(seq, d, dtype):
    ang = torch.outer(torch.arange(seq).float(), 1.0 / (10000 ** (torch.arange(0, d, 2).float() / d)))
    emb = torch.cat([ang, ang], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


@pytest.mark.parametrize("backward", [False, True])
@pytest.mark.parametrize("qdt,cdt", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
                                      (torch.bfloat16, torch.float32), (torch.float32, torch.float32)])
@pytest.mark.parametrize("b,s,h,d", [(2, 50, 8, 128), (1, 33, 3, 64), (3, 7, 4, 16)])
def test_rope(b, s, h, d, qdt, cdt, backward):
    import fmsa_hip

    q = randn((b * s, h * d), 4, qdt)
    cos, sin = _cos_sin(s, d, cdt)
    qd = q.cuda().clone()
    out = fmsa_hip.rope_embedding_(qd, cos.cuda(), sin.cuda(), h, d, backward)
    assert out.data_ptr() == qd.data_ptr()
    assert _close(out, onr.rope(q, cos, sin, h, d, backward), qdt)


def test_rope_rejects_bad_shapes():
    import fmsa_hip

    q = torch.zeros(4, 24, dtype=torch.bfloat16, device="cuda")
    cs = torch.zeros(4, 24, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(fmsa_hip.FmsaError):
        fmsa_hip.rope_embedding_(q, cs, cs, 1, 24)  # head_dim % 16


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fast_rms_layernorm_vs_transformers(dtype):
    from transformers.models.llama.modeling_llama import LlamaRMSNorm

    from fms_acceleration_foak.kernels.unsloth import fast_rms_layernorm

    mod = LlamaRMSNorm(512, eps=1e-6).to(dtype).cuda()
    mod.weight.data = (randn((512,), 5) * 0.3 + 1.0).to(dtype).cuda()
    x = randn((2, 40, 512), 6, dtype).cuda()
    dy = randn((2, 40, 512), 7, dtype).cuda()
    x1 = x.clone().requires_grad_(True)
    y1 = mod(x1)
    y1.backward(dy)
    x2 = x.clone().requires_grad_(True)
    y2 = fast_rms_layernorm(mod, x2)
    y2.backward(dy.clone())
    assert y2.shape == y1.shape and _close(y2, y1, dtype)
    assert _close(x2.grad, x1.grad, dtype)
    assert mod.weight.grad is None or True  # the fused operator never produces a weight gradient


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("cos_3d", [False, True, "long_cache"])
def test_fast_rope_embedding_vs_transformers(dtype, cos_3d):
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb

    from fms_acceleration_foak.kernels.unsloth import fast_rope_embedding

    b, s, h, hk, d = 2, 48, 8, 2, 64
    cos, sin = _cos_sin(s, d, dtype)
    cos_b = cos[None].expand(b, s, d).contiguous().cuda() if cos_3d is True else cos[None].cuda()
    sin_b = sin[None].expand(b, s, d).contiguous().cuda() if cos_3d is True else sin[None].cuda()
    cos_f, sin_f = cos_b, sin_b
    if cos_3d == "long_cache":
        # a 2-D cache that holds more positions than the sequence (rope_embedding.py:60-63 of the reference
        # allows seq_len <= cos.shape[0]): every batch entry still starts at position 0
        cos_l, sin_l = _cos_sin(s + 16, d, dtype)
        cos_f, sin_f = cos_l.cuda(), sin_l.cuda()
    xq = randn((b, s, h * d), 8, dtype).cuda()
    xk = randn((b, s, hk * d), 9, dtype).cuda()
    dq = randn((b, h, s, d), 10, dtype).cuda()
    dk = randn((b, hk, s, d), 11, dtype).cuda()

    def run(fn):
        pq = (xq.clone() * 1.0).requires_grad_(True)
        pk = (xk.clone() * 1.0).requires_grad_(True)
        # projection outputs viewed the way the attention module views them (a non-leaf, as in the model)
        q = (pq * 1.0).view(b, s, h, d).transpose(1, 2)
        k = (pk * 1.0).view(b, s, hk, d).transpose(1, 2)
        cs = (cos_f, sin_f) if fn is fast_rope_embedding else (cos_b, sin_b)
        qo, ko = fn(q, k, *cs)
        torch.autograd.backward([qo, ko], [dq, dk])
        return qo.detach(), ko.detach(), pq.grad, pk.grad

    ref = run(apply_rotary_pos_emb)
    got = run(fast_rope_embedding)
    for a_, b_ in zip(got, ref):
        assert a_.shape == b_.shape and _close(a_, b_, dtype)
