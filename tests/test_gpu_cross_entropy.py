"""Cross-entropy kernels (through the C ABI) against the CPU oracle, and the drop-in loss
functions against torch / transformers.  Tolerance: fp32 arithmetic with hardware exp2 / log2:
1e-5 relative on losses; gradients 1e-5 absolute (softmax entries are <= 1), one storage rounding
on top for 16-bit logits."""
import pytest
import torch
import torch.nn.functional as F

from oracle import cross_entropy as oce
from tests.helpers import randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,V", [(33, 32000), (7, 128256), (5, 50257), (64, 1000), (3, 70003)])
def test_cross_entropy_kernels(M, V, dtype):
    import fmsa_hip

    x = randn((M, V), 1, dtype, scale=3.0)
    y = torch.randint(0, V, (M,), generator=torch.Generator().manual_seed(2))
    y[M // 2] = -100
    y[0], y[-1] = 0, V - 1
    loss, lse = fmsa_hip.cross_entropy_fwd(x.cuda(), y.cuda())
    loss_ref, lse_ref = oce.ce_fwd(x, y)
    assert torch.allclose(loss.cpu(), loss_ref, rtol=2e-5, atol=2e-5)
    assert torch.allclose(lse.cpu(), lse_ref, rtol=2e-5, atol=2e-5)
    assert loss[M // 2].item() == 0.0
    # backward with a per-row dloss and with the expanded scalar of a mean reduction (stride 0)
    for dloss in (torch.rand(M, generator=torch.Generator().manual_seed(3)) + 0.5, torch.tensor(0.25).expand(M)):
        xd = x.cuda().clone()
        g = fmsa_hip.cross_entropy_bwd_(xd, dloss.cuda() if dloss.stride(0) else torch.tensor(0.25, device="cuda").expand(M), lse, y.cuda())
        assert g.data_ptr() == xd.data_ptr()
        g_ref = oce.ce_bwd(x.float(), y, lse_ref, dloss.float())
        tol = 1e-5 if dtype == torch.float32 else (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)
        assert (g.float().cpu() - g_ref).abs().max().item() <= tol * max(1.0, g_ref.abs().max().item())
        assert torch.all(g[M // 2] == 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V", [4096, 1003])
def test_cross_entropy_masked_logits_and_bad_labels(V, dtype):
    """Rows with a masked (-inf) span of the vocabulary -- at the start of the row, where a thread's first
    elements are all -inf, and in the middle -- keep a finite loss and gradient (V = 1003 takes the scalar
    path, V = 4096 the 8-wide one); a label outside [0, V) other than -100 is an ignored row in both passes."""
    import fmsa_hip

    M = 6
    x = randn((M, V), 11, dtype, scale=2.0)
    x[0, :600] = float("-inf")
    x[1, 300:900] = float("-inf")
    x[2, V - 200:] = float("-inf")
    y = torch.tensor([700, 10, 5, V + 3, -7, 2])
    loss, lse = fmsa_hip.cross_entropy_fwd(x.cuda(), y.cuda())
    loss_ref, lse_ref = oce.ce_fwd(x, y)
    assert torch.isfinite(loss).all() and torch.isfinite(lse).all()
    assert torch.allclose(loss.cpu(), loss_ref, rtol=2e-5, atol=2e-5) and torch.allclose(lse.cpu(), lse_ref, rtol=2e-5, atol=2e-5)
    assert loss[3].item() == 0.0 and loss[4].item() == 0.0
    dloss = torch.full((M,), 0.5)
    g = fmsa_hip.cross_entropy_bwd_(x.cuda().clone(), dloss.cuda(), lse, y.cuda())
    g_ref = oce.ce_bwd(x.float(), y, lse_ref, dloss)
    assert torch.isfinite(g).all()
    tol = 1e-5 if dtype == torch.float32 else 2.0 ** -7
    assert (g.float().cpu() - g_ref.float()).abs().max().item() <= tol
    assert torch.all(g[3] == 0) and torch.all(g[4] == 0) and torch.all(g[0, :600] == 0)
    # the fused loss + gradient launch on the same rows (no smoothing: the sum of the logits is not used)
    xf = x.cuda().clone()
    losses, _ = fmsa_hip.cross_entropy_fused_(xf, y.cuda(), scale=None, label_smoothing=0.0)
    assert torch.isfinite(losses).all() and torch.isfinite(xf).all()
    assert torch.allclose(losses.cpu(), loss_ref, rtol=2e-5, atol=2e-5)


def test_fast_cross_entropy_loss_vs_torch():
    from fms_acceleration_foak.kernels.unsloth import FastCrossEntropyLoss, fast_cross_entropy_loss

    b, s, V = 2, 50, 4096
    x = randn((b, s, V), 4, torch.float32, scale=2.0).cuda()
    y = torch.randint(0, V, (b, s), generator=torch.Generator().manual_seed(5)).cuda()
    y[0, :7] = -100
    x1 = x.clone().requires_grad_(True)
    ref = F.cross_entropy(x1.view(-1, V), y.view(-1), ignore_index=-100)
    ref.backward()
    x2 = x.clone().requires_grad_(True)
    got = fast_cross_entropy_loss(x2 * 1.0, y)  # a non-leaf, as in a model (the backward works in place)
    got.backward()
    assert abs(got.item() - ref.item()) < 1e-5 * max(1.0, abs(ref.item()))
    assert torch.allclose(x2.grad, x1.grad, atol=1e-7, rtol=1e-4)
    x3 = x.clone().requires_grad_(True)
    got3 = FastCrossEntropyLoss()((x3 * 1.0).view(-1, V), y.view(-1))
    assert abs(got3.item() - ref.item()) < 1e-5 * max(1.0, abs(ref.item()))


@pytest.mark.parametrize("with_count", [False, True])
def test_fast_for_causal_lm_loss_vs_transformers(with_count):
    from transformers.loss.loss_utils import ForCausalLMLoss

    from fms_acceleration_foak.kernels.unsloth import FastForCausalLMLoss

    b, s, V = 2, 33, 1024
    logits = randn((b, s, V), 6, torch.bfloat16, scale=2.0).cuda()
    labels = torch.randint(0, V, (b, s), generator=torch.Generator().manual_seed(7)).cuda()
    labels[1, 10:] = -100
    kw = {"num_items_in_batch": torch.tensor(40, device="cuda")} if with_count else {}
    l1 = logits.clone().requires_grad_(True)
    ref = ForCausalLMLoss(l1, labels, V, **kw)
    ref.backward()
    l2 = logits.clone().requires_grad_(True)
    got = FastForCausalLMLoss(l2, labels, V, **kw)
    got.backward()
    assert abs(got.item() - ref.item()) < 1e-5 * max(1.0, abs(ref.item()))
    assert torch.allclose(l2.grad.float(), l1.grad.float(), atol=2e-5, rtol=1e-2)
