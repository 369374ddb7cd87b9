"""The fused loss head: `fmsa_cross_entropy_fused` (through the C ABI) against the CPU oracle, the
chunked lm_head + cross-entropy function against the oracle and torch autograd, and `lce_forward` on a
tiny Llama / Granite against the stock forward.  Tolerances: the kernel computes in fp32 with hardware
exp2 / log2 (losses 2e-5 relative; gradients 1e-5 of the scale for fp32 logits, one storage rounding for
16-bit logits); the function adds 16-bit GEMMs, so its gradients are compared at 2^-6 (bf16) / 2^-9 (fp16)
of the largest reference entry."""
import pytest
import torch

from oracle import cross_entropy as oce
from tests.helpers import randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,V,ls,ignore", [(33, 32000, 0.0, -100), (6, 128256, 0.1, -100), (5, 50257, 0.0, 3), (9, 1003, 0.3, -100)])
def test_cross_entropy_fused_kernel(M, V, ls, ignore, dtype):
    import fmsa_hip

    x = randn((M, V), 11, dtype, scale=3.0)
    y = torch.randint(0, V, (M,), generator=torch.Generator().manual_seed(12))
    y[0], y[-1] = 0, V - 1
    y[M // 2] = ignore
    for scale in (None, 1.0 / 7.0):
        xd = x.cuda().clone()
        sc = None if scale is None else torch.tensor([scale], dtype=torch.float32, device="cuda")
        losses, g = fmsa_hip.cross_entropy_fused_(xd, y.cuda(), sc, ls, ignore)
        assert g.data_ptr() == xd.data_ptr()
        loss_ref, g_ref = oce.liger_ce(x, y, 1.0 if scale is None else scale, ls, ignore)
        assert torch.allclose(losses.double().cpu(), loss_ref, rtol=2e-5, atol=2e-5 * (scale or 1.0))
        tol = 1e-5 if dtype == torch.float32 else (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11)
        assert (g.double().cpu() - g_ref).abs().max().item() <= tol * (scale or 1.0)
        assert losses[M // 2].item() == 0.0 and torch.all(g[M // 2] == 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("reduction,ls,with_bias,train_w", [("mean", 0.0, False, False), ("mean", 0.0, False, True),
                                                            ("sum", 0.1, True, True), ("mean", 0.2, True, False)])
def test_fused_linear_cross_entropy_function(reduction, ls, with_bias, train_w, dtype, monkeypatch):
    from fms_acceleration_foak.fused_ops.liger_ce import LigerFusedLinearCrossEntropyLoss
    from fms_acceleration_foak.fused_ops.liger_ce import fused_linear_cross_entropy_loss as mod

    BT, H, V = 300, 256, 2048
    monkeypatch.setattr(mod, "MAX_CHUNK_BYTES", 128 * V * 2)  # several chunks, the last one ragged
    x = randn((BT, H), 21, dtype)
    w = randn((V, H), 22, dtype, scale=H ** -0.5 * 2.0)
    b = randn((V,), 23, dtype) if with_bias else None
    y = torch.randint(0, V, (BT,), generator=torch.Generator().manual_seed(24))
    y[::9] = -100
    xg = x.cuda().requires_grad_(True)
    wg = w.cuda().requires_grad_(train_w)
    bg = None if b is None else b.cuda().requires_grad_(True)
    loss = LigerFusedLinearCrossEntropyLoss(reduction=reduction, label_smoothing=ls)(wg, xg, y.cuda(), bg)
    (loss * 0.5).backward()
    loss_ref, dx, dw, db = oce.fused_linear_ce(x, w, y, b, label_smoothing=ls, reduction=reduction)
    k = {torch.float32: 1e-4, torch.bfloat16: 2.0 ** -6, torch.float16: 2.0 ** -9}[dtype]
    assert loss.dtype == torch.float32 and abs(loss.item() - loss_ref.item()) <= k * abs(loss_ref.item())
    assert xg.grad.dtype == dtype and (xg.grad.double().cpu() - 0.5 * dx).abs().max().item() <= k * 0.5 * dx.abs().max().item()
    if train_w:
        assert (wg.grad.double().cpu() - 0.5 * dw).abs().max().item() <= k * 0.5 * dw.abs().max().item()
    else:
        assert wg.grad is None
    if with_bias:
        assert (bg.grad.double().cpu() - 0.5 * db).abs().max().item() <= k * 0.5 * db.abs().max().item()


def test_fused_linear_cross_entropy_all_ignored_and_autocast():
    from fms_acceleration_foak.fused_ops.liger_ce import LigerFusedLinearCrossEntropyLoss

    x = randn((64, 128), 31, torch.float32).cuda().requires_grad_(True)
    w = randn((512, 128), 32, torch.float32, scale=0.1).cuda().requires_grad_(True)
    y = torch.full((64,), -100, device="cuda")
    loss = LigerFusedLinearCrossEntropyLoss()(w, x, y)
    loss.backward()
    assert loss.item() == 0.0 and float(x.grad.abs().max()) == 0.0 and float(w.grad.abs().max()) == 0.0
    # fp32 master weights under autocast: GEMMs in bf16, gradients come back in the parameters' dtypes
    y = torch.randint(0, 512, (64,), generator=torch.Generator().manual_seed(33)).cuda()
    x.grad = w.grad = None
    with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
        loss = LigerFusedLinearCrossEntropyLoss()(w, x, y)
    loss.backward()
    ref, dx, dw, _ = oce.fused_linear_ce(x.detach().cpu(), w.detach().cpu(), y.cpu())
    assert abs(loss.item() - ref.item()) < 2e-2 * ref.item()
    assert x.grad.dtype == torch.float32 and w.grad.dtype == torch.float32
    assert (x.grad.double().cpu() - dx).abs().max().item() <= 2.0 ** -5 * dx.abs().max().item()
    assert (w.grad.double().cpu() - dw).abs().max().item() <= 2.0 ** -5 * dw.abs().max().item()


@pytest.mark.parametrize("arch", ["llama", "granite"])
@pytest.mark.parametrize("with_count", [False, True])
def test_lce_forward_rule_on_tiny_model(arch, with_count):
    """The `<arch>-fused-lce` rule on a tiny model: same loss and same parameter gradients as the stock
    forward (fp32 model, so only the order of the sums differs), stock behaviour in eval mode."""
    import copy
    import importlib

    from fms_acceleration.model_patcher import ModelPatcher, patch_model
    from fms_acceleration.utils.test_utils import instantiate_model_patcher
    from fms_acceleration_foak.utils import filter_mp_rules

    if arch == "llama":
        from transformers import LlamaConfig as Cfg, LlamaForCausalLM as LM
        extra = {}
    else:
        from transformers import GraniteConfig as Cfg, GraniteForCausalLM as LM
        extra = {"logits_scaling": 4.0}
    torch.manual_seed(0)
    cfg = Cfg(vocab_size=1024, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
              num_key_value_heads=2, max_position_embeddings=64, **extra)
    model = LM(cfg).cuda().train()
    twin = copy.deepcopy(model)
    rules_mod = importlib.import_module(f"fms_acceleration_foak.models.{arch}")
    with instantiate_model_patcher():
        for rule in filter_mp_rules(rules_mod.get_mp_rules("auto_gptq", cfg), {"fused-lce"}):
            ModelPatcher.register(rule)
        patch_model(twin)
        assert [h.rule_id for h in ModelPatcher.history] == [f"{arch}-fused-lce"]
    ids = torch.randint(0, 1024, (3, 17), generator=torch.Generator().manual_seed(1)).cuda()
    labels = ids.clone()
    labels[0, :5] = -100
    kw = {"num_items_in_batch": torch.tensor(40, device="cuda")} if with_count else {}
    out_ref = model(input_ids=ids, labels=labels, **kw)
    out = twin(input_ids=ids, labels=labels, **kw)
    assert out.logits is None and abs(out.loss.item() - out_ref.loss.item()) <= 1e-4 * abs(out_ref.loss.item())
    out_ref.loss.backward()
    out.loss.backward()
    for (n, p), (_, q) in zip(model.named_parameters(), twin.named_parameters()):
        assert q.grad is not None and torch.allclose(q.grad, p.grad, rtol=2e-3, atol=2e-6), n
    twin.eval()
    model.eval()
    with torch.no_grad():
        e_ref, e = model(input_ids=ids, labels=labels), twin(input_ids=ids, labels=labels)
    assert torch.allclose(e.logits, e_ref.logits, atol=1e-5) and abs(e.loss.item() - e_ref.loss.item()) < 1e-5
