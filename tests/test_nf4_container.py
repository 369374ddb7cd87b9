"""Product-side NF4 quantiser / container against the CPU oracle (no GPU needed)."""
import numpy as np
import torch

from oracle import nf4 as onf4


def test_quantize_nf4_matches_oracle():
    from fms_acceleration_peft import quantize_nf4

    rng = np.random.default_rng(0)
    W = (rng.standard_normal((96, 512)) * 0.02).astype(np.float32)
    W[3, :64] = 0.0  # an all-zero block
    packed, st = quantize_nf4(torch.from_numpy(W))
    q = onf4.quantize(W)
    assert np.array_equal(packed.numpy(), q["packed"])
    assert np.array_equal(st.absmax.numpy(), q["absmax_q"])
    assert np.array_equal(st.state2.absmax.numpy(), q["absmax2"])
    assert np.array_equal(st.state2.code.numpy(), q["code2"])
    assert np.array_equal(st.code.numpy(), onf4.NF4)
    assert abs(float(st.offset) - float(q["offset"])) < 1e-7
    assert tuple(st.shape) == (96, 512) and st.blocksize == 64 and st.state2.blocksize == 256


def test_linear4bit_container_and_parameter_scrape():
    from fms_acceleration_foak.fused_ops.unsloth_lora.utils import get_lora_parameters
    from fms_acceleration_peft import Linear4bit, LoraLinear

    base = Linear4bit.from_dense(torch.randn(64, 128) * 0.02, bias=torch.zeros(64))
    assert base.weight.dtype == torch.uint8 and base.weight.shape == (64 * 128 // 2, 1)
    assert not base.weight.requires_grad and base.weight.quant_state.absmax.dtype == torch.uint8
    lin = LoraLinear(base, 8, 16.0)
    W, qs, bias, A, B, s, drop = get_lora_parameters(lin)
    assert W is base.weight and qs is base.weight.quant_state and bias is base.bias
    assert A.shape == (8, 128) and B.shape == (64, 8) and s == 2.0
    lin.enable_adapters(False)
    assert get_lora_parameters(lin)[3:] == (None, None, None, None)


def test_bnb_plugin_shell_and_fused_ops_registry():
    import fms_acceleration  # noqa: F401  (registers the plugins)
    from fms_acceleration_foak.models.utils import FUSED_OPS, KEY_MLP, KEY_O, KEY_QKV
    from fms_acceleration_peft import BNBAccelerationPlugin

    assert set(FUSED_OPS["bitsandbytes"]) == {KEY_QKV, KEY_O, KEY_MLP}
    cfg = {"peft": {"quantization": {"bitsandbytes": {"quant_type": "nf4", "no_peft_model": False}}}}
    plugin = BNBAccelerationPlugin(cfg)
    assert plugin.requires_custom_loading and plugin.requires_augmentation

    class Args:
        bf16, fp16 = True, False

    model = torch.nn.Linear(2, 2)
    plugin.augmentation(model, Args(), (None,))
    assert model.quantization_method == "bitsandbytes"
