"""Pins oracle/cross_entropy.py against torch's own cross entropy and closed forms."""
import math

import torch
import torch.nn.functional as F

from oracle import cross_entropy as oce


def test_forward_matches_torch_and_closed_forms():
    torch.manual_seed(0)
    x = torch.randn(11, 257) * 4.0
    y = torch.randint(0, 257, (11,))
    y[3] = -100
    loss, lse = oce.ce_fwd(x, y)
    ref = F.cross_entropy(x, y, reduction="none", ignore_index=-100)
    assert torch.allclose(loss, ref, rtol=1e-6, atol=1e-6) and loss[3] == 0
    assert torch.allclose(lse, torch.logsumexp(x, dim=-1), rtol=1e-6)
    # uniform logits: loss = log V whatever the label; a shift of the row changes nothing
    u, _ = oce.ce_fwd(torch.full((2, 1000), 3.5), torch.tensor([0, 999]))
    assert torch.allclose(u, torch.full((2,), math.log(1000.0)), rtol=1e-6)
    assert torch.allclose(oce.ce_fwd(x + 100.0, y)[0], loss, atol=1e-4)


def test_backward_matches_autograd():
    torch.manual_seed(1)
    x = (torch.randn(9, 130) * 3.0).double().requires_grad_(True)
    y = torch.randint(0, 130, (9,))
    y[0] = -100
    w = torch.rand(9).double()
    (F.cross_entropy(x, y, reduction="none", ignore_index=-100) * w).sum().backward()
    _, lse = oce.ce_fwd(x.detach(), y)
    g = oce.ce_bwd(x.detach(), y, lse.double(), w)
    assert torch.allclose(g, x.grad, rtol=1e-6, atol=1e-7)
    assert torch.all(g[0] == 0) and torch.allclose(g.sum(-1), torch.zeros(9).double(), atol=1e-6)


def test_liger_ce_matches_torch_with_label_smoothing():
    import pytest

    torch.manual_seed(2)
    for ls, ignore in ((0.0, -100), (0.1, -100), (0.35, 7)):
        x = (torch.randn(13, 97) * 3.0).double().requires_grad_(True)
        y = torch.randint(0, 97, (13,))
        y[2] = ignore
        y[9] = ignore
        ref = F.cross_entropy(x, y, reduction="none", ignore_index=ignore, label_smoothing=ls)
        (ref.sum() * 0.25).backward()
        loss, g = oce.liger_ce(x.detach(), y, 0.25, ls, ignore)
        assert loss.tolist() == pytest.approx((ref.detach() * 0.25).tolist(), rel=1e-10, abs=1e-12)
        assert torch.allclose(g, x.grad, rtol=1e-10, atol=1e-12)
        assert torch.all(g[2] == 0) and loss[9] == 0
    # full smoothing on uniform logits: the loss is log V and the gradient vanishes
    loss, g = oce.liger_ce(torch.full((1, 50), -2.0), torch.tensor([4]), 1.0, 1.0)
    assert abs(float(loss) - math.log(50.0)) < 1e-12 and float(g.abs().max()) < 1e-15


def test_fused_linear_ce_matches_autograd():
    torch.manual_seed(3)
    for reduction, ls, with_bias in (("mean", 0.0, False), ("sum", 0.2, True), ("mean", 0.1, True)):
        x = torch.randn(10, 24).double().requires_grad_(True)
        w = torch.randn(40, 24).double().requires_grad_(True)
        b = torch.randn(40).double().requires_grad_(True) if with_bias else None
        y = torch.randint(0, 40, (10,))
        y[5] = -100
        ref = F.cross_entropy(F.linear(x, w, b), y, reduction=reduction, label_smoothing=ls)
        ref.backward()
        loss, dx, dw, db = oce.fused_linear_ce(x.detach(), w.detach(), y, None if b is None else b.detach(),
                                               label_smoothing=ls, reduction=reduction)
        assert abs(float(loss) - float(ref.detach())) < 1e-10
        assert torch.allclose(dx, x.grad, rtol=1e-9, atol=1e-12) and torch.allclose(dw, w.grad, rtol=1e-9, atol=1e-12)
        assert (db is None) == (b is None) and (b is None or torch.allclose(db, b.grad, rtol=1e-9, atol=1e-12))
    # every label ignored under a mean reduction: zero loss and gradients, not NaN
    loss, dx, dw, _ = oce.fused_linear_ce(torch.randn(3, 8), torch.randn(5, 8), torch.full((3,), -100))
    assert float(loss) == 0 and float(dx.abs().max()) == 0 and float(dw.abs().max()) == 0


def test_masked_logits_and_labels_outside_the_vocabulary():
    """-inf logits (a masked span) give the logsumexp of the rest, as torch's own loss does; a label outside [0, V)
    is an ignored row (loss 0, zero gradient), like -100."""
    V = 37
    x = torch.randn(4, V, generator=torch.Generator().manual_seed(1)) * 2
    x[0, :10] = float("-inf")
    x[1, 20:] = float("-inf")
    y = torch.tensor([12, 3, V + 5, -100])
    loss, lse = oce.ce_fwd(x, y)
    ref = F.cross_entropy(x[:2], y[:2], reduction="none")
    assert torch.allclose(loss[:2], ref, atol=1e-6) and loss[2] == 0 and loss[3] == 0
    assert torch.allclose(lse, torch.logsumexp(x, dim=-1), atol=1e-6)
    g = oce.ce_bwd(x, y, lse, torch.ones(4))
    assert torch.isfinite(g).all() and torch.all(g[2] == 0) and torch.all(g[3] == 0) and torch.all(g[0, :10] == 0)
    assert torch.allclose(g[:2].sum(dim=-1), torch.zeros(2), atol=1e-6)
