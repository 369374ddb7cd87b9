"""GPTQ checkpoint format: config round trip with the reference's synonyms, v1 <-> v2 zero points
(checked through the oracle's dequantisation), and loading a saved tiny Llama into QuantLinears."""
import json

import numpy as np
import pytest
import torch

from oracle import gptq as ogptq
from tests.helpers import make_gptq


def test_quantize_config_round_trip_and_synonyms(tmp_path):
    from fms_acceleration_peft import QuantizeConfig

    cfg = QuantizeConfig(bits=4, group_size=128, desc_act=False, sym=False, format="gptq_v2")
    cfg.save_pretrained(str(tmp_path))
    raw = json.load(open(tmp_path / "quantize_config.json"))
    assert raw["checkpoint_format"] == "gptq_v2" and "format" not in raw
    back = QuantizeConfig.from_pretrained(str(tmp_path))
    assert back == cfg
    old = QuantizeConfig.from_quant_config({"w_bit": 4, "q_group_size": 64, "version": "GEMM"})
    assert old.bits == 4 and old.group_size == 64 and old.format == "gptq"  # no format field: v1
    with pytest.raises(ValueError):
        QuantizeConfig(bits=5)
    # transformers-style config.json
    (tmp_path / "sub").mkdir()
    json.dump({"quantization_config": {"bits": 4, "group_size": 32, "checkpoint_format": "gptq"}}, open(tmp_path / "sub" / "config.json", "w"))
    assert QuantizeConfig.from_pretrained(str(tmp_path / "sub")).group_size == 32


def test_v1_v2_zero_points_are_the_same_weight():
    from fms_acceleration_peft import QuantizeConfig, QuantLinear, convert_gptq_v1_to_v2_format, convert_gptq_v2_to_v1_format

    w = make_gptq(256, 64, 64, seed=1)
    ql = QuantLinear(4, 64, 256, 64, False)
    ql.load_packed(w["np"]["qweight"], w["np"]["qzeros"], w["np"]["scales"], w["np"]["g_idx"])
    holder = torch.nn.Sequential(ql)
    cfg = QuantizeConfig(bits=4, group_size=64)
    v2 = ql.qzeros.clone()
    convert_gptq_v2_to_v1_format(holder, cfg)
    assert np.array_equal(ql.qzeros.numpy(), ogptq.to_v1_zeros(np.ascontiguousarray(v2.numpy())))
    dense_v1 = ogptq.dequant(w["np"]["qweight"], w["np"]["scales"], ql.qzeros.numpy(), w["np"]["g_idx"], zero_offset=1, out="fp32")
    assert torch.equal(dense_v1, w["dense"])  # v1 zeros + offset 1 == v2 zeros
    convert_gptq_v1_to_v2_format(holder, cfg)
    assert torch.equal(ql.qzeros, v2)


@pytest.mark.parametrize("fmt", ["gptq", "gptq_v2"])
def test_save_and_load_tiny_llama(tmp_path, fmt):
    from transformers import LlamaConfig, LlamaForCausalLM

    from fms_acceleration_peft import QuantizeConfig, QuantLinear, load_quantized, save_quantized
    from fms_acceleration_peft.quantizer import quantize_linear

    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=64)
    torch.manual_seed(0)
    model = LlamaForCausalLM(cfg)
    dense = {}
    for name, mod in list(model.named_modules()):
        if isinstance(mod, torch.nn.Linear) and "lm_head" not in name:
            ql = quantize_linear(mod.weight.data, 32)
            dense[name] = ogptq.dequant_torch(ql.qweight, ql.scales, ql.qzeros, ql.g_idx)
            parent = model.get_submodule(name.rsplit(".", 1)[0])
            setattr(parent, name.rsplit(".", 1)[1], ql)
    qcfg = QuantizeConfig(bits=4, group_size=32, desc_act=False, sym=False, format=fmt)
    save_quantized(model, str(tmp_path), qcfg)

    fresh = LlamaForCausalLM(cfg)
    loaded, got = load_quantized(fresh, str(tmp_path))
    assert got.format == "gptq_v2" and loaded.quantization_method == "gptq"
    qls = {n: m for n, m in loaded.named_modules() if isinstance(m, QuantLinear)}
    assert set(qls) == set(dense) and len(qls) == 7
    for n, m in qls.items():
        assert torch.equal(ogptq.dequant_torch(m.qweight, m.scales, m.qzeros, m.g_idx), dense[n]), n
    assert torch.equal(loaded.lm_head.weight, model.lm_head.weight)
    assert torch.equal(loaded.model.embed_tokens.weight, model.model.embed_tokens.weight)
    # a model that does not match the file is refused
    other = LlamaForCausalLM(LlamaConfig(hidden_size=64, intermediate_size=128, num_attention_heads=4, num_key_value_heads=2,
                                         num_hidden_layers=2, vocab_size=64))
    with pytest.raises(KeyError):
        load_quantized(other, str(tmp_path))


def test_plugin_model_loader_reads_a_local_directory(tmp_path):
    from transformers import LlamaConfig, LlamaForCausalLM

    from fms_acceleration_peft import AutoGPTQAccelerationPlugin, QuantizeConfig, QuantLinear, save_quantized
    from fms_acceleration_peft.quantizer import quantize_linear

    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=64)
    cfg.architectures = ["LlamaForCausalLM"]
    model = LlamaForCausalLM(cfg)
    for name, mod in list(model.named_modules()):
        if isinstance(mod, torch.nn.Linear) and "lm_head" not in name:
            setattr(model.get_submodule(name.rsplit(".", 1)[0]), name.rsplit(".", 1)[1], quantize_linear(mod.weight.data, 32))
    save_quantized(model, str(tmp_path), QuantizeConfig(bits=4, group_size=32, desc_act=False, sym=False))
    cfg.save_pretrained(str(tmp_path))
    plugin = AutoGPTQAccelerationPlugin({"peft": {"quantization": {"auto_gptq": {"kernel": "triton_v2", "from_quantized": True}}}})
    loaded = plugin.model_loader(str(tmp_path), torch_dtype=torch.float16, device="cpu")
    assert loaded.quantization_method == "gptq"
    assert sum(isinstance(m, QuantLinear) for m in loaded.modules()) == 7
    assert loaded.lm_head.weight.dtype == torch.float16
    with pytest.raises(NotImplementedError):
        plugin.model_loader("TheBloke/Llama-2-7B-GPTQ")


def test_augmentation_installs_adapters_and_the_fused_rules_trigger(tmp_path):
    """model_loader -> AutoGPTQ augmentation (adapters from a duck-typed peft_config) -> fast-kernels augmentation
    -> ModelPatcher: the qkvo and mlp rules fire on the adapted modules (reference: the LoRA layers come from
    get_gptq_peft_model, framework_plugin_autogptq.py:250-330, and the triggers look for lora_A / lora_B / base_layer,
    fused-ops-and-kernels models/utils.py:46-49,195-204)."""
    from transformers import LlamaConfig, LlamaForCausalLM

    from fms_acceleration.model_patcher import ModelPatcher, patch_model
    from fms_acceleration.utils.test_utils import instantiate_model_patcher
    from fms_acceleration_foak import FastKernelsAccelerationPlugin
    from fms_acceleration_peft import AutoGPTQAccelerationPlugin, LoraLinear, QuantizeConfig, QuantLinear, save_quantized
    from fms_acceleration_peft.quantizer import quantize_linear

    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=2, vocab_size=64)
    cfg.architectures = ["LlamaForCausalLM"]
    model = LlamaForCausalLM(cfg)
    for name, mod in list(model.named_modules()):
        if isinstance(mod, torch.nn.Linear) and "lm_head" not in name:
            setattr(model.get_submodule(name.rsplit(".", 1)[0]), name.rsplit(".", 1)[1], quantize_linear(mod.weight.data, 32))
    save_quantized(model, str(tmp_path), QuantizeConfig(bits=4, group_size=32, desc_act=False, sym=False))
    cfg.save_pretrained(str(tmp_path))
    plugin = AutoGPTQAccelerationPlugin({"peft": {"quantization": {"auto_gptq": {"kernel": "triton_v2", "from_quantized": True}}}})
    loaded = plugin.model_loader(str(tmp_path), torch_dtype=torch.float16, device="cpu")
    train_args = type("T", (), {"bf16": False, "fp16": True, "gradient_checkpointing": False})()

    with pytest.raises(AssertionError, match="peft_config"):
        plugin.augmentation(loaded, train_args, (None,))
    with pytest.raises(ValueError, match="no QuantLinear module matches"):
        plugin.augmentation(loaded, train_args, ({"r": 8, "lora_alpha": 16, "target_modules": ["no_such_proj"]},))

    peft_config = type("LoraConfig", (), {"r": 8, "lora_alpha": 16, "lora_dropout": 0.0,
                                          "target_modules": ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]})()
    out, args = plugin.augmentation(loaded, train_args, (peft_config,))
    assert out is loaded and args == (None,)
    wrapped = [m for m in loaded.modules() if isinstance(m, LoraLinear)]
    assert len(wrapped) == 14 and all(isinstance(m.base_layer, QuantLinear) and m.scaling["default"] == 2.0 for m in wrapped)
    trainable = [n for n, p in loaded.named_parameters() if p.requires_grad]
    assert len(trainable) == 28 and all("lora_" in n for n in trainable)

    foak = FastKernelsAccelerationPlugin({"training": {"fused_ops_and_kernels": {"fused_lora": True, "base_layer": "auto_gptq"}}})
    with instantiate_model_patcher():
        foak.augmentation(loaded, train_args, ())
        patch_model(loaded)
        done = {h.rule_id for h in ModelPatcher.history}
        assert "llama-mlp" in done and any(d.startswith("llama-qkvo") for d in done)
        assert sum(h.rule_id == "llama-mlp" for h in ModelPatcher.history) == 2   # one per decoder layer
