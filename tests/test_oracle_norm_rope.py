"""Pins oracle/norm_rope.py against independent statements: transformers' LlamaRMSNorm and
apply_rotary_pos_emb (library code), autograd, and closed forms."""
import pytest
import torch

from oracle import norm_rope as onr


def test_rms_fwd_matches_transformers_and_unit_rms():
    from transformers.models.llama.modeling_llama import LlamaRMSNorm

    torch.manual_seed(0)
    x = torch.randn(7, 96) * 3.0
    mod = LlamaRMSNorm(96, eps=1e-5)
    mod.weight.data = torch.randn(96)
    y, r = onr.rms_fwd(x, mod.weight.data, 1e-5)
    assert torch.allclose(y, mod(x), rtol=1e-6, atol=1e-6)
    # with unit weight every output row has rms 1 (up to eps)
    y1, _ = onr.rms_fwd(x, torch.ones(96), 0.0)
    assert torch.allclose(y1.pow(2).mean(-1), torch.ones(7), atol=1e-5)
    assert torch.allclose(r, 1.0 / x.pow(2).mean(-1).sqrt(), rtol=1e-5)
    # bf16 input: statistics in fp32, the product rounded in the weight's dtype (HF does the same)
    xb, wb = x.bfloat16(), mod.weight.data.bfloat16()
    modb = LlamaRMSNorm(96, eps=1e-5).bfloat16()
    modb.weight.data = wb
    assert torch.equal(onr.rms_fwd(xb, wb, 1e-5)[0], modb(xb))


@pytest.mark.parametrize("gemma", [False, True])
def test_rms_bwd_matches_autograd(gemma):
    torch.manual_seed(1)
    x = torch.randn(5, 64, dtype=torch.float64, requires_grad=True)
    w = torch.randn(64, dtype=torch.float64)
    dy = torch.randn(5, 64, dtype=torch.float64)
    weff = w + 1.0 if gemma else w
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * weff
    y.backward(dy)
    _, r = onr.rms_fwd(x.detach().float(), w.float(), 1e-6, gemma)
    dx = onr.rms_bwd(dy.float(), x.detach().float(), w.float(), r, gemma)
    assert torch.allclose(dx.double(), x.grad, rtol=1e-4, atol=1e-5)
    if gemma:  # gemma forward: weight + 1 in fp32
        yg, _ = onr.rms_fwd(x.detach().float(), w.float(), 1e-6, True)
        assert torch.allclose(yg.double(), y.detach(), rtol=1e-5, atol=1e-6)


def test_rope_matches_transformers_and_is_a_rotation():
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb

    torch.manual_seed(2)
    b, s, h, d = 2, 9, 3, 32
    q = torch.randn(b, h, s, d)
    k = torch.randn(b, h, s, d)
    inv_freq = 1.0 / (10000 ** (torch.arange(0, d, 2).float() / d))
    ang = torch.outer(torch.arange(s).float(), inv_freq)
    emb = torch.cat([ang, ang], dim=-1)
    cos, sin = emb.cos(), emb.sin()  # [s, d]
    q_ref, k_ref = apply_rotary_pos_emb(q, k, cos[None], sin[None])
    flat = lambda t: t.transpose(1, 2).reshape(b * s, h * d)  # noqa: E731
    q_or = onr.rope(flat(q), cos, sin, h, d)
    k_or = onr.rope(flat(k), cos, sin, h, d)
    assert torch.allclose(q_or, flat(q_ref), atol=1e-6) and torch.allclose(k_or, flat(k_ref), atol=1e-6)
    # a rotation: norms per (token, head) are preserved, and the backward pass (sin negated) inverts it
    assert torch.allclose(q_or.view(b * s, h, d).norm(dim=-1), flat(q).view(b * s, h, d).norm(dim=-1), rtol=1e-5)
    assert torch.allclose(onr.rope(q_or, cos, sin, h, d, backward=True), flat(q), atol=1e-5)
    # position 0 is the identity
    assert torch.allclose(q_or.view(b, s, h * d)[:, 0], flat(q).view(b, s, h * d)[:, 0], atol=1e-7)


def test_rope_backward_is_the_vjp():
    torch.manual_seed(3)
    s, h, d = 6, 2, 16
    q = torch.randn(s, h * d, dtype=torch.float64, requires_grad=True)
    ang = torch.outer(torch.arange(s).double(), 1.0 / (10000 ** (torch.arange(0, d, 2).double() / d)))
    cos, sin = torch.cat([ang, ang], -1).cos(), torch.cat([ang, ang], -1).sin()
    half = d // 2
    qh = q.view(s, h, d)
    c, sn = cos[:, None, :half], sin[:, None, :half]
    out = torch.cat([qh[..., :half] * c - qh[..., half:] * sn, qh[..., half:] * c + qh[..., :half] * sn], -1).view(s, h * d)
    dy = torch.randn(s, h * d, dtype=torch.float64)
    out.backward(dy)
    assert torch.allclose(onr.rope(dy.float(), cos.float(), sin.float(), h, d, backward=True).double(), q.grad, atol=1e-5)


def test_rope_table_rows_of_the_host_wrapper():
    """The table the kernel indexes with (token row % rows): a 2-D cache longer than the sequence is cut to
    seq_len rows, so batch entry b restarts at position 0 (reference rope_embedding.py:60-63: row % seq_len
    with seq_len <= cos.shape[0]); a per-batch 3-D table is flattened row by row."""
    import pytest

    from fms_acceleration_foak.kernels.unsloth.rope_embedding import _rows

    b, s, h, d = 2, 5, 2, 16
    ang = torch.outer(torch.arange(s + 3).float(), 1.0 / (10000 ** (torch.arange(0, d, 2).float() / d)))
    cache = torch.cat([ang, ang], -1).cos()
    for form in (cache, cache[None]):
        t = _rows(form, b, s)
        assert t.shape == (s, d) and torch.equal(t, cache[:s])
    per_batch = torch.stack([cache[:s], cache[3:3 + s]])
    assert torch.equal(_rows(per_batch, b, s), per_batch.reshape(b * s, d))
    with pytest.raises(ValueError):
        _rows(cache[: s - 1], b, s)
    with pytest.raises(ValueError):
        _rows(per_batch[:, : s - 1], b, s)
    # with that table the oracle's row % rows lookup gives batch 1 the positions 0 .. s-1 again
    q = torch.randn(b * s, h * d, generator=torch.Generator().manual_seed(3))
    sin = torch.cat([ang, ang], -1).sin()
    out = onr.rope(q, _rows(cache, b, s), _rows(sin, b, s), h, d)
    assert torch.allclose(out[s:], onr.rope(q[s:], cache[:s], sin[:s], h, d))
