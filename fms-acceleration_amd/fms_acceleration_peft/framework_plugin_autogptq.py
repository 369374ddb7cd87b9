"""Configuration shell of the GPTQ-LoRA plugin (reference:
accelerated-peft/src/fms_acceleration_peft/framework_plugin_autogptq.py:44-395).

Only the boundary is built: registration under `peft.quantization.auto_gptq`, validation of the
configuration keys, and the `quantization_method` marker that the fast-kernels plugin keys on.
Loading a quantised checkpoint and installing PEFT adapters need the gptqmodel loader, peft and
hub checkpoints; callers of this build construct `QuantLinear` + `LoraLinear` modules directly.
"""
from fms_acceleration import AccelerationPlugin


class AutoGPTQAccelerationPlugin(AccelerationPlugin):
    require_packages = []

    def __init__(self, configurations):
        super().__init__(configurations)
        self._check_config_equal(key="peft.quantization.auto_gptq.kernel", value="triton_v2")
        self._check_config_equal(key="peft.quantization.auto_gptq.from_quantized", value=True)
        self.use_external_lib = self._check_config_and_maybe_check_values(
            key="peft.quantization.auto_gptq.use_external_lib", values=[True, False], default=False
        )

    @property
    def requires_custom_loading(self):
        return True

    @property
    def requires_augmentation(self):
        return True

    def model_loader(self, model_name: str, **kwargs):
        raise NotImplementedError(
            "GPTQ checkpoint loading is outside the fused-LoRA hot path of this build: wrap the "
            "model's linears in fms_acceleration_peft.QuantLinear / LoraLinear and set "
            "model.quantization_method = 'gptq'"
        )

    def augmentation(self, model, train_args, modifiable_args):
        # the marker FastKernelsAccelerationPlugin.augmentation looks for (:235-236 of the reference)
        setattr(model, "quantization_method", "gptq")
        return model, modifiable_args


AccelerationPlugin.register_plugin(AutoGPTQAccelerationPlugin, configuration_and_paths=["peft.quantization.auto_gptq"])
