"""Configuration shell of the bitsandbytes-LoRA plugin (reference:
accelerated-peft/src/fms_acceleration_peft/framework_plugin_bnb.py:95-260).

Only the boundary is built: registration under `peft.quantization.bitsandbytes`, validation of
`quant_type` / `no_peft_model`, the mixed-precision assertion of `augmentation`, and the
`quantization_method` marker.  Checkpoint loading through transformers' BitsAndBytesConfig and PEFT
adapter installation are not part of the fused-LoRA hot path; callers of this build construct
`Linear4bit` + `LoraLinear` modules directly.  Only `nf4` has a kernel.
"""
from fms_acceleration import AccelerationPlugin


class BNBAccelerationPlugin(AccelerationPlugin):
    require_packages = []

    def __init__(self, configurations):
        super().__init__(configurations)
        self._quant_type = self._check_config_and_maybe_check_values(
            key="peft.quantization.bitsandbytes.quant_type", values=["fp4", "nf4"]
        )
        self._no_peft_model = self._check_config_and_maybe_check_values(
            key="peft.quantization.bitsandbytes.no_peft_model", values=[True, False]
        )
        if self._quant_type != "nf4":
            raise NotImplementedError("only quant_type 'nf4' has a dequantisation kernel in this build")

    @property
    def requires_custom_loading(self):
        return True

    @property
    def requires_augmentation(self):
        return not self._no_peft_model

    def model_loader(self, model_name: str, **kwargs):
        raise NotImplementedError(
            "NF4 checkpoint loading is outside the fused-LoRA hot path of this build: wrap the model's "
            "linears in fms_acceleration_peft.Linear4bit / LoraLinear and set "
            "model.quantization_method = 'bitsandbytes'"
        )

    def augmentation(self, model, train_args, modifiable_args):
        assert (
            getattr(train_args, "bf16", False) is True or getattr(train_args, "fp16", False) is True
        ), f"{self.__class__} requires mixed precision argument `--fp16` or `--bf16`"
        setattr(model, "quantization_method", "bitsandbytes")
        return model, modifiable_args


AccelerationPlugin.register_plugin(BNBAccelerationPlugin, configuration_and_paths=["peft.quantization.bitsandbytes"])
