"""QuantLinear's own forward / backward (base projection only, fused dequant-GEMM kernels with the
adapter disabled) against the oracle's dense weight, and an end-to-end check: a GPTQ checkpoint on
disk -> local loader -> LoRA wrappers -> plugin patch rules -> one forward/backward of a tiny
Llama, against the same model run without any patching."""
import copy

import pytest
import torch

from oracle import lora as olora
from tests.helpers import make_gptq, randn

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("K,N,gs", [(512, 256, 128), (352, 96, 32), (256, 64, 16)])
def test_quantlinear_forward_backward(K, N, gs, act_order, dtype):
    from fms_acceleration_peft import QuantLinear

    w = make_gptq(K, N, gs, seed=2, act_order=act_order)
    ql = QuantLinear(4, gs, K, N, True)
    ql.load_packed(w["np"]["qweight"], w["np"]["qzeros"], w["np"]["scales"], w["np"]["g_idx"])
    ql.bias.copy_((randn((N,), 5) * 0.1).half())
    ql = ql.cuda()
    x = randn((3, 40, K), 1, dtype)
    dy = randn((3, 40, N), 2, dtype)
    xg = x.cuda().requires_grad_(True)
    y = ql(xg)
    y.backward(dy.cuda())
    y_ref = x.float() @ w["dense"] + ql.bias.float().cpu()
    dx_ref = dy.float() @ w["dense"].t()
    assert y.dtype == dtype and y.shape == (3, 40, N)
    assert olora.max_rel_err(y.reshape(-1, N), y_ref.reshape(-1, N)) < TOL
    assert olora.max_rel_err(xg.grad.reshape(-1, K), dx_ref.reshape(-1, K)) < TOL


# rope: True = the reference's separate fast_rope_embedding pass after the fused projections; "fused_qkv" = Q and K
# rotated inside the fused projection launch
@pytest.mark.parametrize("rope", [True, "fused_qkv"])
def test_checkpoint_to_patched_training_step(tmp_path, rope, monkeypatch):
    import fmsa_hip
    from transformers import LlamaConfig, LlamaForCausalLM

    from fms_acceleration.model_patcher import ModelPatcher, patch_model
    from fms_acceleration.utils.test_utils import instantiate_model_patcher
    from fms_acceleration_foak import FastKernelsAccelerationPlugin
    from fms_acceleration_peft import AutoGPTQAccelerationPlugin, LoraLinear, QuantizeConfig, QuantLinear, save_quantized
    from fms_acceleration_peft.quantizer import quantize_linear
    import transformers.models.llama.modeling_llama as ml

    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=2, vocab_size=128, attention_dropout=0.0)
    cfg.architectures = ["LlamaForCausalLM"]
    cfg._attn_implementation = "eager"
    torch.manual_seed(0)
    src = LlamaForCausalLM(cfg)
    for name, mod in list(src.named_modules()):
        if isinstance(mod, torch.nn.Linear) and "lm_head" not in name:
            setattr(src.get_submodule(name.rsplit(".", 1)[0]), name.rsplit(".", 1)[1], quantize_linear(mod.weight.data, 64))
    save_quantized(src, str(tmp_path), QuantizeConfig(bits=4, group_size=64, desc_act=False, sym=False))
    cfg.save_pretrained(str(tmp_path))

    loader = AutoGPTQAccelerationPlugin({"peft": {"quantization": {"auto_gptq": {"kernel": "triton_v2", "from_quantized": True}}}})
    model = loader.model_loader(str(tmp_path), torch_dtype=torch.bfloat16, device="cuda")
    # LoRA on every quantised linear, B made non-zero so the adapters matter
    gen = torch.Generator().manual_seed(1)
    for name, mod in list(model.named_modules()):
        if isinstance(mod, QuantLinear):
            lin = LoraLinear(mod, 8, 16.0).cuda()
            lin.lora_B["default"].weight.data.copy_(torch.randn(lin.lora_B["default"].weight.shape, generator=gen) * 0.05)
            setattr(model.get_submodule(name.rsplit(".", 1)[0]), name.rsplit(".", 1)[1], lin)
    for n, p in model.named_parameters():  # what PEFT does: only the adapters train
        p.requires_grad_("lora_" in n)
    plain = copy.deepcopy(model)

    ids = torch.randint(0, 128, (2, 64), generator=torch.Generator().manual_seed(3)).cuda()

    def step(m):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = m(input_ids=ids, labels=ids)
        out.loss.backward()
        grads = {n: p.grad.float().clone() for n, p in m.named_parameters() if p.grad is not None}
        return out.loss.item(), grads

    loss_ref, grads_ref = step(plain)
    plugin = FastKernelsAccelerationPlugin({"training": {"fused_ops_and_kernels": {
        "fused_lora": True, "fast_loss": True, "fast_rms_layernorm": True, "fast_rope_embeddings": rope}}})
    seen = {"fwd_with_rope": 0, "rope_fwd_pass": 0, "rope_bwd_pass": 0}
    real_fwd, real_rope = fmsa_hip.gptq_lora_fwd, fmsa_hip.rope_embedding_

    def count_fwd(*a, **k):
        seen["fwd_with_rope"] += k.get("rope") is not None
        return real_fwd(*a, **k)

    def count_rope(*a, backward=False, **k):
        seen["rope_bwd_pass" if backward else "rope_fwd_pass"] += 1
        return real_rope(*a, backward=backward, **k)

    monkeypatch.setattr(fmsa_hip, "gptq_lora_fwd", count_fwd)
    monkeypatch.setattr(fmsa_hip, "rope_embedding_", count_rope)
    original = ml.apply_rotary_pos_emb
    try:
        with instantiate_model_patcher():
            plugin.augmentation(model, type("T", (), {"bf16": True, "fp16": False})(), ())
            patch_model(model)
            done = {h.rule_id for h in ModelPatcher.history}
            assert {"llama-mlp", "llama-rms", "llama-rope", "llama-custom-loss"} <= done
            assert any(d.startswith("llama-qkvo") for d in done) and model.loss_type == "llama-custom-loss"
            loss, grads = step(model)
    finally:
        ml.apply_rotary_pos_emb = original
    # per layer: one forward launch that rotates Q and K and no separate forward pass, or two separate passes
    assert seen == ({"fwd_with_rope": 2, "rope_fwd_pass": 0, "rope_bwd_pass": 4} if rope == "fused_qkv"
                    else {"fwd_with_rope": 0, "rope_fwd_pass": 4, "rope_bwd_pass": 4})
    assert abs(loss - loss_ref) < 2e-2 * max(1.0, abs(loss_ref))
    assert set(grads) == set(grads_ref) and len(grads) == 2 * 7 * 2  # lora_A and lora_B of 7 projections x 2 layers
    worst = max(olora.max_rel_err(grads[n], grads_ref[n]) for n in grads)
    assert worst < 5e-2, worst
